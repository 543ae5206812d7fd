// A sequence of decode linears (M <= 4 tokens) in ONE persistent launch, layout L1.
// HBM-bandwidth bound: algorithmic bytes = sum over the linears of
// N*K/2 + (K/g)*N*4 + M*K*2 + M*N*2.
//
// Why.  A decode linear of 9..36 MB takes 1..4.5 us of HBM time, but a kernel launch that depends on
// its predecessor costs about 2.5 us on this part before its first byte arrives (an empty kernel in a
// chain of dependent launches takes that long), and drains its tail with the memory system idle.
// Weight addresses do not depend on the previous linear's output: only the activations do.  This
// kernel keeps one workgroup resident per CU for the whole sequence; its streaming waves run one
// weight stream across all linears, and while a linear waits for activations that other workgroups
// are still producing, the stream goes on into a ring in LDS.
//
// Roles.  A workgroup has 8 streaming waves and 4 control waves; there is no workgroup barrier in the
// kernel, the two kinds of waves meet through counters in LDS.
//   Streaming waves request weights (global -> LDS direct loads into a private ring of 1 KiB slots,
//   one slot per wave-wide 128-bit load), multiply them with the activations staged in LDS and leave
//   partial sums in LDS.  They never wait for anything in memory but their own oldest load, and they
//   bound the number of loads they keep in flight: vector memory operations of a CU return in order,
//   so everything a control wave asks for queues behind what the streaming waves have outstanding.
//   While the activations of the next linear are not there yet, a streaming wave keeps filling its
//   ring (waiting for its oldest load before it issues another) until the ring is full.
//   Control waves own everything that needs a wait on memory: they sum the partial sums, apply the
//   epilogue, store Y, publish it to the other workgroups and stage the next linear's activations.
//
// Exchange between workgroups (no grid barrier).  A linear whose output is read by a later linear of
// the same launch (as activations or residual: the pointers are compared) also stores it to the
// workspace as 8-byte words {two fp16 values, 32-bit tag} with one device-coherent (sc1) store per
// word; the tag is the launch's number, kept in the workspace and advanced by the last wave to leave.
// A consumer reads those words with sc1 loads and repeats the read until every tag is the launch's:
// data and flag arrive in one aligned 8-byte access, so a dependency costs one store and one load
// instead of store, wait, counter, poll and load.  Polls are bounded; when one runs out, a sticky
// error word is set and the launch finishes with undefined results instead of hanging.
//
// Mapping (arithmetic as in the single-linear GEMV).  v_mfma_f32_4x4x4_16B_f16 multiplies 16
// independent 4x4x4 blocks; in block b lane 4b+i supplies row i of A (tokens) and column i of B
// (weights of output row i) and receives D[0..3][i].  A wave-wide 128-bit load covers 4 rows x 256
// contiguous bytes = 4 rows x 512 k (a step).  Workgroup g owns the rows [g*R, (g+1)*R) of every
// linear (R = ceil(N / workgroups) rounded up to 4), cut into units of 4 rows x 2048 k (four steps);
// unit u goes to streaming wave u % 8.  The zeros/scales of a unit (4 rows x 2048/g groups) are one
// to four direct loads whose neighbouring lanes are neighbours in memory.
//
// Activations: the whole [M, K] input of the current linear is staged in LDS (K <= 16384: 32 KiB per
// token) with the per-32-k sums the zero-point fixup needs; row pitch K*2 + 16 bytes keeps the 64
// lanes of a 128-bit read on distinct slots.
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
constexpr int SEQ_S = 4;                          // steps (128-bit loads per lane) per unit
constexpr int SEQ_KSUB = 512 * SEQ_S;
constexpr int SEQ_USLOTS_MAX = 7;                 // unit slots of a wave's ring: their loads fit the 6-bit counter

typedef unsigned long long u64;

struct SeqLinear {
    const uint8_t* w;
    const half2_t* zs;
    const half_t* x;
    half_t* y;
    const half_t* bias;
    const half_t* residual;
    const u64* xsrc;   // the activations as exchange words of an earlier linear of this launch, or null
    const u64* rsrc;   // the residual as exchange words, or null
    u64* ydst;         // where this linear publishes its output for later linears, or null
    int N, K, gshift, act;
    int rows;     // rows per workgroup (multiple of 4)
    int nch;      // units per row group = ceil(K / 2048)
    int units;    // units per workgroup = rows / 4 * nch
    int kpad;     // K rounded up to 2048
    int stage;    // how many stagings of activations have happened when this linear's are in LDS
    int restage;  // 1: the control waves stage activations for this linear
    int red_off;  // float offset of this linear's partial sums in LDS
    int need;     // streaming waves that have units of this linear
};

struct SeqArgs {
    SeqLinear p[SEQ_MAX_LINEARS];
    int count;
    int M;
    unsigned* ctrl;       // workspace control block: [0] launch number, [1] sticky error word, [2] exit counter
    unsigned spin_limit;
    int xsum_off;         // byte offsets of the LDS regions behind the activations
    int red_off;
    int sync_off;         // [0] stagings completed x control waves, [1 + l] streaming waves done with linear l
    int ring_off;         // first wave's ring; per wave: uslots x 4 KiB of weights, then uslots x zbytes
    int ring_stride;
    int uslots;
    int zbytes;           // bytes of one zeros/scales slot = 256 nz
    int nz;               // zeros/scales loads per unit = 2048 / group size / 16 (all linears share the group size)
    int lim;              // units a streaming wave keeps in flight (1 or 2; 3 only counts as 2 when it waits)
};


__device__ __forceinline__ void load_to_lds_nt_x4(const void* g, uint32_t lds_byte) {
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(g), "{m0}"(lds_byte) : "memory");
}

// A value read from the argument buffer, pinned in scalar registers: without this the compiler, knowing the buffer
// never changes, re-reads a field wherever it is used (a scalar load and a wait of a few hundred cycles each time).
template <typename T>
__device__ __forceinline__ T pinned(T v) {
    asm volatile("" : "+s"(v));
    return v;
}

__device__ __forceinline__ int lds_counter(const int* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }

// ---------------------------------------------------------------------------------------- streaming waves
// The units of wave `wave` in order: for every linear l, u = wave, wave + 8, ... < units; rg = u / nch is the
// unit's row group, c = u % nch its 2048-wide piece of K.
struct UnitCursor {
    int l, u, rg, c;
};
// First linear at or behind cur.l in which this wave has a unit (cur.u = wave on entry to a new linear).
__device__ __forceinline__ void cursor_place(const SeqArgs& a, int count, UnitCursor& cur, int wave) {
    while (cur.l < count && cur.u >= pinned(a.p[cur.l].units)) {
        cur.l++;
        cur.u = wave;
    }
}
// One unit on inside a linear of `units` units and `nch` pieces of K; false when the linear is exhausted.
__device__ __forceinline__ bool cursor_step(UnitCursor& cur, int units, int nch) {
    cur.u += SEQ_SW;
    if (cur.u >= units) return false;
    cur.c += SEQ_SW;
    while (cur.c >= nch) {
        cur.c -= nch;
        cur.rg++;
    }
    return true;
}

// Wait until at most n units' worth of this wave's loads are outstanding (n = 0, 1 or 2; a unit is 4 + nz loads).
__device__ __forceinline__ void wait_units(int n, int nz) {
    if (n <= 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else if (n == 1) {
        if (nz == 1) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
        else if (nz == 2) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    } else {
        if (nz == 1) asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
        else if (nz == 2) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    }
}

template <int MROWS>
__device__ __forceinline__ void streaming_wave(const SeqArgs& a, uint8_t* lds, int wave, int wg) {
    const NibbleMasks nm = nibble_masks();
    const int lane = threadIdx.x & 63;
    const int i = lane & 3;
    const int b = lane >> 2;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const int uslots = pinned(a.uslots);
    const int zbytes = pinned(a.zbytes);
    const uint32_t wring = pinned(a.ring_off + wave * a.ring_stride);  // unit slots of 4 KiB, then their zeros/scales slots
    const uint32_t zring = wring + uslots * 4096;
    const uint8_t* xbuf = lds;
    const float* xsum = (const float*)(lds + a.xsum_off);
    int* sync = (int*)(lds + a.sync_off);
    const int nz = pinned(a.nz);
    const int lim = pinned(a.lim);
    const int red_base = pinned(a.red_off);

    // The counters in LDS start at zero; the one workgroup barrier of the kernel separates that from their first
    // use, and lets the control waves' first activation loads into the memory pipeline ahead of the weights.
    if (wave == 0 && lane < 1 + SEQ_MAX_LINEARS) sync[lane] = 0;
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    const int count = pinned(a.count);
    UnitCursor ic = {0, wave, 0, 0}, cc = {0, wave, 0, 0};  // issue side, consume side
    cursor_place(a, count, ic, wave);
    cc = ic;
    // the linears at the two cursors, kept in scalar registers (the argument buffer is read on a change only)
    struct Pinned {
        const uint8_t* w;
        const uint32_t* zs;
        int N, K, gshift, rows, nch, units, kpad, stage, red_off;
    };
    auto fetch = [&a](int l) {
        const SeqLinear& q = a.p[l];
        return Pinned{pinned(q.w), pinned((const uint32_t*)q.zs), pinned(q.N), pinned(q.K), pinned(q.gshift), pinned(q.rows),
                      pinned(q.nch), pinned(q.units), pinned(q.kpad), pinned(q.stage), pinned(q.red_off)};
    };
    Pinned Li = fetch(ic.l < count ? ic.l : 0);
    ic.rg = ic.u / Li.nch;
    ic.c = ic.u - ic.rg * Li.nch;
    cc = ic;
    Pinned Lc = Li;
    int u_issued = 0, u_consumed = 0;  // units requested / multiplied so far
    int u_returned = 0;                // units known to have arrived
    int slot_i = 0, slot_c = 0;        // ring slots at the two cursors
    int staged = 0;                    // last value read of the staging counter

    while (cc.l < count) {
        // ---- request: as long as there is a free slot and the wave is within its in-flight allowance
        while (ic.l < count && u_issued - u_consumed < uslots && u_issued - u_returned < lim) {
            const Pinned& L = Li;
            const int row0 = wg * L.rows + 4 * ic.rg;
            {
                // zeros/scales of the unit: lane 16 r + q fetches group q + 16 t of row r
                const int gpu_ = SEQ_KSUB >> L.gshift;  // groups per unit and row
                const int groups = L.K >> L.gshift;
                const int zr = imin(row0 + (lane >> 4), L.N - 1);
                const uint32_t* zrow = L.zs + (long)zr * groups;
                const uint32_t zslot = lds0 + zring + slot_i * zbytes;
                for (int t = 0; t < nz; t++) {
                    const int gi = ic.c * gpu_ + 16 * t + (lane & 15);
                    load_to_lds_x1(zrow + (gi < groups ? gi : 0), zslot + t * 256);
                }
            }
            const int row = imin(row0 + i, L.N - 1);
            const uint8_t* wrow = L.w + (long)row * (L.K >> 1);
            const int k0 = ic.c * SEQ_KSUB + 32 * b;
            const uint32_t wslot = lds0 + wring + slot_i * 4096;
#pragma unroll
            for (int st = 0; st < SEQ_S; st++) {
                const int kk = k0 + 512 * st;
                load_to_lds_nt_x4(wrow + ((kk < L.K ? kk : 0) >> 1), wslot + st * 1024);
            }
            u_issued++;
            slot_i = slot_i + 1 == uslots ? 0 : slot_i + 1;
            if (!cursor_step(ic, L.units, L.nch)) {
                ic.l++;
                ic.u = wave;
                cursor_place(a, count, ic, wave);
                if (ic.l < count) {
                    Li = fetch(ic.l);
                    ic.rg = ic.u / Li.nch;
                    ic.c = ic.u - ic.rg * Li.nch;
                }
            }
        }
        // ---- are the activations of the linear at the consume cursor in LDS?
        const Pinned& L = Lc;
        if (staged < SEQ_CW * L.stage) staged = __builtin_amdgcn_readfirstlane(lds_counter(&sync[0]));
        if (staged >= SEQ_CW * L.stage) {
            // wait for the unit's loads (zeros/scales first, then the four steps)
            if (u_returned <= u_consumed) {
                wait_units(u_issued - u_consumed - 1, nz);
                u_returned = u_consumed + 1;
            }
            const int pitch = L.kpad * 2 + 16;
            const uint8_t* wslot = lds + wring + slot_c * 4096 + lane * 16;
            const uint8_t* zslot = lds + zring + slot_c * zbytes + 64 * i;
            const int kb0 = cc.c * SEQ_KSUB + 32 * b;
            const uint8_t* xp0 = xbuf + (i & (MROWS - 1)) * pitch + kb0 * 2;
            const float* xs0 = xsum + (kb0 >> 5) * MROWS * 2;
            u32x4_t wq[SEQ_S];
            half2_t zq[SEQ_S];
#pragma unroll
            for (int st = 0; st < SEQ_S; st++) {
                wq[st] = *(const u32x4_t*)(wslot + st * 1024);
                const int gi = (512 * st + 32 * b) >> L.gshift;
                zq[st] = *(const half2_t*)(zslot + (gi >> 4) * 256 + (gi & 15) * 4);
            }
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int st = 0; st < SEQ_S; st++) {
                half8_t xa[4];
#pragma unroll
                for (int q = 0; q < 4; q++) xa[q] = *(const half8_t*)(xp0 + 1024 * st + 16 * q);
                float4_t tmp = {0.f, 0.f, 0.f, 0.f}, tmp2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const half8_t wv = unpack8_mixed(wq[st][q], nm);
                    float4_t& tq = q < 2 ? tmp : tmp2;
                    tq = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[q].lo, wv.lo, tq, 0, 0, 0);
                    tq = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[q].hi, wv.hi, tq, 0, 0, 0);
                }
                tmp += tmp2;
                const float zf = (float)zq[st].x;
                const float sf = (float)zq[st].y;
                const float* xs = xs0 + 16 * st * MROWS * 2;
#pragma unroll
                for (int m = 0; m < MROWS; m++) acc[m] += sf * ((tmp[m] - xs[2 * m + 1]) - zf * xs[2 * m]);
            }
            // fold the 16 blocks of the wave; lanes 0..3 hold rows 4*rg + 0..3
            float* red = (float*)(lds + red_base) + L.red_off;
#pragma unroll
            for (int m = 0; m < MROWS; m++) {
                float v = row_sum_stride4(acc[m]);
                v += __shfl_xor(v, 16);
                v += __shfl_xor(v, 32);
                if (lane < 4) red[(cc.u * MROWS + m) * 4 + i] = v;
            }
            u_consumed++;
            slot_c = slot_c + 1 == uslots ? 0 : slot_c + 1;
            if (!cursor_step(cc, L.units, L.nch)) {
                // this wave's last unit of the linear: its partial sums are in LDS before the count moves
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (lane == 0) __hip_atomic_fetch_add(&sync[1 + cc.l], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                cc.l++;
                cc.u = wave;
                cursor_place(a, count, cc, wave);
                if (cc.l < count) {
                    Lc = fetch(cc.l);
                    cc.rg = cc.u / Lc.nch;
                    cc.c = cc.u - cc.rg * Lc.nch;
                }
            }
        } else if (u_issued > u_returned && ic.l < count && u_issued - u_consumed < uslots) {
            // not yet: make room in the in-flight allowance by waiting for the oldest outstanding unit
            wait_units(u_issued - u_returned - 1, nz);
            u_returned++;
        } else {
            __builtin_amdgcn_s_sleep(2);
        }
    }
}

// ---------------------------------------------------------------------------------------- control waves
// Eight device-coherent 128-bit loads, the workgroup barrier of the kernel's start, then the wait for the loads:
// the streaming waves are released as soon as these requests are on their way, so that the weight requests
// queue up behind them and not in front of them.
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
        "s_waitcnt lgkmcnt(0)\n\t"
        "s_barrier\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7])
        : "memory");
}

// Activations from memory the launch does not write: [M, K] fp16, zero beyond M and K.
template <int MROWS>
__device__ __forceinline__ void stage_plain(const SeqLinear& L, int M, uint8_t* xbuf, float* xsum, int ct,
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

// Activations that an earlier linear of this launch publishes: exchange words {fp16 y[m][2j], fp16 y[m][2j+1], tag}
// at xsrc[m * K/2 + j].  A thread takes eight consecutive values (four words, two 128-bit loads) and four such
// items per trip; the trip is repeated until every tag in the wave is the launch's.  Returns false when the
// polls ran out.
template <int MROWS>
__device__ __forceinline__ bool stage_exchange(const SeqLinear& L, int M, uint8_t* xbuf, float* xsum, int ct,
                                               unsigned tag, unsigned spin_limit) {
    const int pitch = L.kpad * 2 + 16;
    const int items_per_row = L.kpad >> 3;  // eight values each
    const int items = MROWS * items_per_row;
    bool all_ok = true;
    for (int base = 0; base < items; base += 4 * SEQ_CT) {
        const float* ptr[8];
        float4_t v[8];
        int mm[4], ww[4];
        bool ok[4], in[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int idx = base + q * SEQ_CT + ct;
            mm[q] = idx / items_per_row;
            ww[q] = idx - mm[q] * items_per_row;
            in[q] = idx < items;
            ok[q] = in[q] && mm[q] < M && ww[q] * 8 < L.K;
            const u64* src = L.xsrc + (ok[q] ? (long)mm[q] * (L.K >> 1) + ww[q] * 4 : 0);
            ptr[2 * q] = (const float*)src;
            ptr[2 * q + 1] = (const float*)(src + 2);
        }
        unsigned polls = 0;
        for (;;) {
            load8_coherent_x4(ptr, v);
            bool good = true;
#pragma unroll
            for (int q = 0; q < 4; q++)
                if (ok[q]) {
                    const u32x4_t a0 = bit_cast<u32x4_t>(v[2 * q]), a1 = bit_cast<u32x4_t>(v[2 * q + 1]);
                    good = good && a0.y == tag && a0.w == tag && a1.y == tag && a1.w == tag;
                }
            if (__builtin_amdgcn_ballot_w64(!good) == 0) break;
            if (++polls > spin_limit) {
                all_ok = false;
                break;
            }
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const u32x4_t a0 = bit_cast<u32x4_t>(v[2 * q]), a1 = bit_cast<u32x4_t>(v[2 * q + 1]);
            u32x4_t packed = {a0.x, a0.z, a1.x, a1.z};
            if (!ok[q]) packed = (u32x4_t){0u, 0u, 0u, 0u};
            const half8_t h = bit_cast<half8_t>(packed);
            float lo = ((float)h[0] + (float)h[1]) + ((float)h[4] + (float)h[5]);
            float sum = lo + (((float)h[2] + (float)h[3]) + ((float)h[6] + (float)h[7]));
            sum = quad_sum(sum);
            lo = quad_sum(lo);
            if (in[q]) {
                *(u32x4_t*)(xbuf + mm[q] * pitch + ww[q] * 16) = packed;
                if ((ct & 3) == 0) {
                    float* xs = xsum + ((ww[q] >> 2) * MROWS + mm[q]) * 2;
                    xs[0] = sum;
                    xs[1] = 960.f * lo;
                }
            }
        }
    }
    return all_ok;
}

__device__ __forceinline__ u64 load_word_coherent(const u64* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int MROWS>
__device__ __forceinline__ void control_wave(const SeqArgs& a, uint8_t* lds, int ct, int wg, int nwg) {
    uint8_t* xbuf = lds;
    float* xsum = (float*)(lds + a.xsum_off);
    int* sync = (int*)(lds + a.sync_off);
    const int M = a.M;
    const int count = a.count;
    // the launch's tag: one more than the number the previous launch on this workspace left behind
    const unsigned tag = __hip_atomic_load(&a.ctrl[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
    bool failed = false;
    stage_plain<MROWS>(a.p[0], M, xbuf, xsum, ct, true);  // contains the workgroup barrier of the kernel's start
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if ((ct & 63) == 0) __hip_atomic_fetch_add(&sync[0], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);

    for (int cl = 0; cl < count; cl++) {
        const SeqLinear& L = a.p[cl];
        // this thread's outputs: token m, rows 2 rp and 2 rp + 1 of the workgroup's (one exchange word)
        const int half_rows = L.rows >> 1;
        const int items = half_rows * MROWS;
        // Bias and residual are requested before the wait for the streaming waves (one item per thread covers
        // every decoder shape; further items fetch theirs late).
        const int m0 = ct / half_rows, rp0 = ct - m0 * half_rows;
        const int n00 = wg * L.rows + 2 * rp0;
        const bool first_ok = ct < items && n00 < L.N && m0 < M;
        uint32_t bias0 = 0;
        u64 res0 = 0;
        if (first_ok && L.bias) bias0 = *(const uint32_t*)(L.bias + n00);
        if (first_ok && L.residual)
            res0 = L.rsrc ? load_word_coherent(L.rsrc + (((long)m0 * L.N + n00) >> 1))
                          : (u64) * (const uint32_t*)(L.residual + (long)m0 * L.N + n00) | ((u64)tag << 32);
        // every streaming wave with units of this linear has left its partial sums
        while (lds_counter(&sync[1 + cl]) < L.need) __builtin_amdgcn_s_sleep(1);
        const float* red = (const float*)(lds + a.red_off) + L.red_off;
        for (int t = ct; t < items; t += SEQ_CT) {
            const int m = t / half_rows;
            const int rp = t - m * half_rows;
            const int n0 = wg * L.rows + 2 * rp;
            if (n0 < L.N && m < M) {
                float v[2];
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const int r = 2 * rp + e;
                    const float* pr = red + ((r >> 2) * L.nch * MROWS + m) * 4 + (r & 3);
                    float s = 0.f;
                    for (int c = 0; c < L.nch; c++) s += pr[c * MROWS * 4];  // fixed order: bit-reproducible
                    v[e] = s;
                }
                if (L.bias) {
                    const half2_t bb = bit_cast<half2_t>(t == ct ? bias0 : *(const uint32_t*)(L.bias + n0));
                    v[0] += (float)bb.x;
                    v[1] += (float)bb.y;
                }
                if (L.act == 1) {
                    v[0] = fmaxf(v[0], 0.f);
                    v[1] = fmaxf(v[1], 0.f);
                }
                if (L.residual) {
                    u64 rw = res0;
                    if (t != ct)
                        rw = L.rsrc ? load_word_coherent(L.rsrc + (((long)m * L.N + n0) >> 1))
                                    : (u64) * (const uint32_t*)(L.residual + (long)m * L.N + n0) | ((u64)tag << 32);
                    unsigned polls = 0;
                    while ((unsigned)(rw >> 32) != tag) {  // only a residual this launch produces can fail the test
                        if (++polls > a.spin_limit) {
                            failed = true;
                            break;
                        }
                        rw = load_word_coherent(L.rsrc + (((long)m * L.N + n0) >> 1));
                    }
                    const half2_t rr = bit_cast<half2_t>((uint32_t)rw);
                    v[0] += (float)rr.x;
                    v[1] += (float)rr.y;
                }
                const half2_t out = {(half_t)v[0], (half_t)v[1]};
                const uint32_t bits = bit_cast<uint32_t>(out);
                if (L.ydst) {
                    const u32x2_t word = {bits, tag};
                    asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(L.ydst + (((long)m * L.N + n0) >> 1)), "v"(word)
                                 : "memory");
                }
                *(uint32_t*)(L.y + (long)m * L.N + n0) = bits;
            }
        }
        if (cl + 1 < count && a.p[cl + 1].restage) {
            const SeqLinear& Ln = a.p[cl + 1];
            if (Ln.xsrc) {
                if (!stage_exchange<MROWS>(Ln, M, xbuf, xsum, ct, tag, a.spin_limit)) failed = true;
            } else {
                stage_plain<MROWS>(Ln, M, xbuf, xsum, ct);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if ((ct & 63) == 0) __hip_atomic_fetch_add(&sync[0], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
    if (__builtin_amdgcn_ballot_w64(failed) != 0 && (ct & 63) == 0)
        __hip_atomic_store(&a.ctrl[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // Exit: the last control wave of the launch to get here advances the launch number (every poll of this
    // launch is over by then) and clears the exit counter.
    if ((ct & 63) == 0) {
        const unsigned old = __hip_atomic_fetch_add(&a.ctrl[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old == (unsigned)(nwg * SEQ_CW - 1)) {
            __hip_atomic_store(&a.ctrl[2], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&a.ctrl[0], tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

template <int MROWS>
__global__ __launch_bounds__(SEQ_NT) void gemv_seq_kernel(const SeqArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (wave >= SEQ_SW)
        control_wave<MROWS>(a, lds, tid - 64 * SEQ_SW, blockIdx.x, gridDim.x);
    else
        streaming_wave<MROWS>(a, lds, wave, blockIdx.x);
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

template <int MROWS>
hipError_t launch_m(const SeqArgs& a, int grid, size_t lds_bytes, hipStream_t st) {
    static bool attr_set[64] = {};
    int dev = 0;
    (void)hipGetDevice(&dev);
    auto kern = gemv_seq_kernel<MROWS>;
    if (dev >= 0 && dev < 64 && !attr_set[dev]) {
        const hipError_t e =
            hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SEQ_LDS_LIMIT);
        if (e != hipSuccess) return e;
        attr_set[dev] = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(SEQ_NT), lds_bytes, st, a);
    return hipGetLastError();
}

constexpr size_t SEQ_XCHG_OFF = 256;  // the control block comes first

inline bool overlaps(const void* a, size_t na, const void* b, size_t nb) {
    if (!a || !b) return false;
    const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
    return pa < pb + nb && pb < pa + na;
}

// Which earlier linear of the list writes the buffer `p` (exactly: same address, same extent)?  -1: none.
inline int producer_of(const SeqProblem* probs, int l, const void* p, size_t bytes, int M) {
    for (int q = l - 1; q >= 0; q--)
        if (probs[q].y == p && (size_t)M * probs[q].N * 2 == bytes) return q;
    return -1;
}

// The data flow of the list as this kernel can honour it: src_x[l] / src_r[l] = the linear that produces the
// activations / the residual of linear l inside the launch (-1: memory the launch does not write).  False when the
// list has a hazard the kernel has no ordering for (the caller then launches the linears one by one).
bool plan_flow(const SeqProblem* probs, int count, int M, int* src_x, int* src_r) {
    for (int l = 0; l < count; l++) {
        const SeqProblem& q = probs[l];
        const size_t xb = (size_t)M * q.K * 2, yb = (size_t)M * q.N * 2;
        src_x[l] = producer_of(probs, l, q.x, xb, M);
        src_r[l] = q.residual ? producer_of(probs, l, q.residual, yb, M) : -1;
        if (q.depends && src_x[l] < 0 && src_r[l] < 0) return false;  // depends on something this kernel cannot see
        // every workgroup has finished linear `fence` (and all reads of the linears up to it) before any
        // workgroup can store an output of linear l
        const int fence = src_x[l] > src_r[l] ? src_x[l] : src_r[l];
        for (int p = 0; p <= l; p++) {
            const SeqProblem& e = probs[p];
            const size_t exb = (size_t)M * e.K * 2, eyb = (size_t)M * e.N * 2;
            const bool reads = overlaps(q.y, yb, e.x, exb) || overlaps(q.y, yb, e.residual, eyb);
            if (reads && p > fence) return false;                       // a write that may overtake a read
            if (p < l && overlaps(q.y, yb, e.y, eyb)) return false;     // two linears writing one buffer
            // partial overlaps of a read with an earlier output are not the exact match producer_of() wants
            if (p < l && src_x[l] != p && overlaps(q.x, xb, e.y, eyb)) return false;
            if (p < l && src_r[l] != p && overlaps(q.residual, yb, e.y, eyb)) return false;
        }
        if (src_x[l] >= 0 && probs[src_x[l]].N != q.K) return false;
        // the halves of an exchange word and the 32-bit accesses of the tail
        if ((reinterpret_cast<uintptr_t>(q.bias) & 3u) || (reinterpret_cast<uintptr_t>(q.residual) & 3u)) return false;
    }
    return true;
}


}  // namespace


size_t gemv_seq_workspace_bytes(const SeqProblem* probs, int count, int M) {
    size_t need = SEQ_XCHG_OFF;
    if (!probs || count < 1 || count > SEQ_MAX_LINEARS || M < 1 || M > 4) return need;
    int src_x[SEQ_MAX_LINEARS], src_r[SEQ_MAX_LINEARS];
    if (!plan_flow(probs, count, M, src_x, src_r)) return need;
    bool published[SEQ_MAX_LINEARS] = {};
    for (int l = 0; l < count; l++) {
        if (src_x[l] >= 0) published[src_x[l]] = true;
        if (src_r[l] >= 0) published[src_r[l]] = true;
    }
    for (int l = 0; l < count; l++)
        if (published[l]) need += (((size_t)M * probs[l].N * 4) + 255) & ~(size_t)255;
    return need;
}

int launch_gemv_seq(const SeqProblem* probs, int count, int M, void* workspace, size_t workspace_bytes,
                    unsigned spin_limit, int lim, hipStream_t st) {
    if (count < 1 || count > SEQ_MAX_LINEARS || M < 1 || M > 4) return 1;
    if (!workspace || workspace_bytes < gemv_seq_workspace_bytes(probs, count, M)) return 1;
    const int grid = cu_count();
    if (grid <= 0) return 2;
    int src_x[SEQ_MAX_LINEARS], src_r[SEQ_MAX_LINEARS];
    if (!plan_flow(probs, count, M, src_x, src_r)) return 1;
    const int mrows = M <= 1 ? 1 : (M <= 2 ? 2 : 4);
    SeqArgs a;
    a.count = count;
    a.M = M;
    a.ctrl = (unsigned*)workspace;
    a.spin_limit = spin_limit;
    int kpad_max = 0, red_floats = 0, stage = 0;
    size_t xchg = SEQ_XCHG_OFF;
    u64* dst[SEQ_MAX_LINEARS] = {};
    for (int l = 0; l < count; l++) {
        bool published = false;
        for (int c = l + 1; c < count; c++) published = published || src_x[c] == l || src_r[c] == l;
        if (published) {
            dst[l] = (u64*)((uint8_t*)workspace + xchg);
            xchg += (((size_t)M * probs[l].N * 4) + 255) & ~(size_t)255;
        }
    }
    for (int l = 0; l < count; l++) {
        const SeqProblem& q = probs[l];
        if (q.group_size != probs[0].group_size) return 1;
        if (q.N % 2 != 0) return 1;
        SeqLinear& L = a.p[l];
        L.w = (const uint8_t*)q.w;
        L.zs = (const half2_t*)q.zs;
        L.x = (const half_t*)q.x;
        L.y = (half_t*)q.y;
        L.bias = (const half_t*)q.bias;
        L.residual = (const half_t*)q.residual;
        L.xsrc = src_x[l] >= 0 ? dst[src_x[l]] : nullptr;
        L.rsrc = src_r[l] >= 0 ? dst[src_r[l]] : nullptr;
        L.ydst = dst[l];
        L.N = q.N;
        L.K = q.K;
        L.gshift = 0;
        while ((1 << L.gshift) < q.group_size) L.gshift++;
        L.act = q.act;
        L.rows = (((q.N + grid - 1) / grid) + 3) & ~3;
        L.kpad = ((q.K + SEQ_KSUB - 1) / SEQ_KSUB) * SEQ_KSUB;
        L.nch = L.kpad / SEQ_KSUB;
        L.units = (L.rows / 4) * L.nch;
        L.need = L.units < SEQ_SW ? L.units : SEQ_SW;
        L.restage = (l == 0 || q.x != probs[l - 1].x || q.K != probs[l - 1].K) ? 1 : 0;
        if (L.restage) stage++;
        L.stage = stage;
        L.red_off = red_floats;
        red_floats += L.units * mrows * 4;
        if (L.kpad > kpad_max) kpad_max = L.kpad;
    }
    for (int l = count; l < SEQ_MAX_LINEARS; l++) a.p[l] = a.p[0];
    a.nz = (SEQ_KSUB >> a.p[0].gshift) / 16;
    if (a.nz < 1) return 1;
    a.zbytes = 256 * a.nz;
    const size_t xbuf_bytes = (size_t)mrows * ((size_t)kpad_max * 2 + 16);
    const size_t xsum_bytes = (size_t)(kpad_max / 32) * mrows * 2 * sizeof(float);
    a.xsum_off = (int)((xbuf_bytes + 15) & ~(size_t)15);
    a.red_off = (int)((a.xsum_off + xsum_bytes + 15) & ~(size_t)15);
    a.sync_off = (int)((a.red_off + (size_t)red_floats * sizeof(float) + 15) & ~(size_t)15);
    a.ring_off = (a.sync_off + 64 + 1023) & ~1023;
    if ((size_t)a.ring_off + 1024 > SEQ_LDS_LIMIT) return 1;
    const size_t per_wave = (SEQ_LDS_LIMIT - a.ring_off) / SEQ_SW;
    a.uslots = (int)(per_wave / (4096 + a.zbytes));
    if (a.uslots < 2) return 1;  // less than two units per wave: not worth a persistent launch
    if (a.uslots > SEQ_USLOTS_MAX) a.uslots = SEQ_USLOTS_MAX;
    a.ring_stride = a.uslots * (4096 + a.zbytes);
    a.lim = lim > 0 ? lim : 1;
    if (a.lim > 2) a.lim = 2;
    if (a.lim > a.uslots - 1) a.lim = a.uslots - 1;
    const size_t lds_bytes = (size_t)a.ring_off + (size_t)SEQ_SW * a.ring_stride;
    const hipError_t e = mrows == 1 ? launch_m<1>(a, grid, lds_bytes, st)
                                    : (mrows == 2 ? launch_m<2>(a, grid, lds_bytes, st) : launch_m<4>(a, grid, lds_bytes, st));
    return e == hipSuccess ? 0 : 2;
}

}  // namespace sq
