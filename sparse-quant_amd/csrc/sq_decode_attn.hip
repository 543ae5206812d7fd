// Dense decode attention: one query token per sequence against an fp16 key/value cache,
// optionally appending the step's new key/value row to the cache in the same launch.
//
// out[b,h,:] = sum_j P[j] * V[b,h,j,:],  P = softmax_j(q[b,h,:] . K[b,h,j,:] * sm_scale + mask[b,j])
// over the rows j < L of the cache, fp32 softmax and accumulation, fp16 output -- the decode
// branch of the reference's sparse_attention
// (reference: sparse-attention/nvidia/playground/kernels/block_sparse_attention_lut.py:272-300).
//
// The work is a pure stream over the cache (2 * L * D * 2 bytes per head, two flops per
// byte), so the kernel is laid out for the memory system and nothing else:
//   * one workgroup of eight waves per (batch, head); a wave's 128-bit load covers 64/(D/8)
//     consecutive cache rows = 1 KiB of contiguous memory (eight whole 128-byte lines); the K
//     and V rows of a batch of rows are requested together, the next batch while the current
//     one is consumed;
//   * one pass: every 16-lane (D = 128) or 8-lane (D = 64) row slot of every wave runs its own
//     online softmax (running maximum, sum and 8 output columns per lane, all fp32) over the
//     rows it is dealt; no barrier and no LDS inside the stream; the 32 or 64 partial states
//     of a head are merged once at the end.  The probabilities meet V unrounded (the reference
//     rounds the normalised ones to fp16 first; the difference is below its own rounding);
//   * the row that is being appended is taken from the new-row pointers, never read back from
//     the cache, and stored to the cache by the lanes that hold it.
// The number of valid rows may live on the device (HIP-graph replay with a growing cache).
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

namespace {

constexpr int DA_WAVES = 8;
constexpr int DA_U = 4;  // rows of a batch per row slot: 128-bit loads per wave and operand in one request (6 and 8: no faster)

struct DecodeAttnArgs {
    const half_t* q;
    const half_t* kn;
    const half_t* vn;
    half_t* kc;
    half_t* vc;
    const half_t* mask;
    half_t* o;
    long q_bs, q_hs;  // element strides of q over batch / head
    long n_bs, n_hs;  // ... of the new key and value rows
    long c_bs, c_hs;  // ... of both caches (row stride is D)
    long m_bs;        // ... of the additive mask over batch
    int H, Lmax, cache_len;
    const long long* cache_len_dev;
    float scale;
    // Split of the cache rows over gridDim.y workgroups per (batch, head), for launches with too few
    // heads to fill the chip: partial softmax states (m, l, D outputs) meet in `part`, one counter
    // per head in `counters` (zero between calls), the last arriver merges.
    float* part;
    unsigned* counters;
};

__device__ __forceinline__ float xor_sum(float v, int m) { return v + __shfl_xor(v, m, 64); }

template <int D, bool MASK>
__global__ __launch_bounds__(64 * DA_WAVES) void decode_attn_kernel(DecodeAttnArgs a) {
    constexpr int LPR = D / 8;    // lanes per cache row
    constexpr int RPI = 64 / LPR; // rows per load instruction
    constexpr int STEP = DA_WAVES * RPI * DA_U;
    __shared__ float mred[DA_WAVES];
    __shared__ float lred[DA_WAVES];
    __shared__ float ored[DA_WAVES][D];
    __shared__ unsigned last_flag;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: the stream's loop is then uniform control flow
    const int c = lane % LPR;
    const int r = lane / LPR;
    const int b = blockIdx.x / a.H;
    const int h = blockIdx.x % a.H;
    const bool append = a.kn != nullptr;

    int n0 = a.cache_len_dev ? (int)*a.cache_len_dev : a.cache_len;
    const int n0max = a.Lmax - (append ? 1 : 0);
    n0 = n0 < 0 ? 0 : (n0 > n0max ? n0max : n0);
    const int L = n0 + (append ? 1 : 0);  // rows attended; the appended row is row n0
    // This workgroup's share of the rows: [r0, r1).
    const int nsplit = gridDim.y;
    const int rows_per = (L + nsplit - 1) / nsplit;
    const int r0 = imin(blockIdx.y * rows_per, L);
    const int r1 = imin(r0 + rows_per, L);

    half_t* kbase = a.kc + (long)b * a.c_bs + (long)h * a.c_hs + 8 * c;
    half_t* vbase = a.vc + (long)b * a.c_bs + (long)h * a.c_hs + 8 * c;
    const half_t* knrow = append ? a.kn + (long)b * a.n_bs + (long)h * a.n_hs + 8 * c : nullptr;
    const half_t* vnrow = append ? a.vn + (long)b * a.n_bs + (long)h * a.n_hs + 8 * c : nullptr;
    const half_t* mrow = a.mask ? a.mask + (long)b * a.m_bs : nullptr;
    const half8_t qv = *(const half8_t*)(a.q + (long)b * a.q_bs + (long)h * a.q_hs + 8 * c);
    const half2_t q01 = {qv[0], qv[1]}, q23 = {qv[2], qv[3]}, q45 = {qv[4], qv[5]}, q67 = {qv[6], qv[7]};

    // Row j of a batch that starts at `base`: base + u * RPI + r (clamped for the loads; rows past
    // the end get probability zero).
    auto load_rows = [&](const half_t* cache, const half_t* fresh, int base, u32x4_t (&dst)[DA_U]) {
#pragma unroll
        for (int u = 0; u < DA_U; u++) {
            const int j = imin(base + u * RPI + r, r1 - 1);
            const half_t* src = (append && j == n0) ? fresh : cache + (long)j * D;
            dst[u] = __builtin_nontemporal_load((const u32x4_t*)src);
        }
    };
    // The appended row goes into the cache once, up front, by the lanes of the workgroup whose share holds it
    // (the stream below takes it from the new-row pointers and never reads it back).
    if (append && n0 >= r0 && n0 < r1 && wave == 0 && r == 0) {
        *(u32x4_t*)(kbase + (long)n0 * D) = *(const u32x4_t*)knrow;
        *(u32x4_t*)(vbase + (long)n0 * D) = *(const u32x4_t*)vnrow;
    }

    // Online softmax state of this lane's row slot (the LPR lanes of a slot hold the same m and l).
    float m = -INFINITY, l = 0.f;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.f;

    // The stream.  No branch and no store inside the loop: the next batch of rows is always requested (row
    // indices clamped to the share, so a batch past the end re-reads the last row and gets probability zero),
    // which keeps the compiler's wait counts exact: the arithmetic of a batch waits for that batch only while
    // the next one is in flight.
    u32x4_t ka[DA_U], va[DA_U], kb[DA_U], vb[DA_U];
    float ma[DA_U], mb_[DA_U];
    auto load_mask = [&](int base, float (&dst)[DA_U]) {
#pragma unroll
        for (int u = 0; u < DA_U; u++) dst[u] = MASK ? (float)mrow[imin(base + u * RPI + r, r1 - 1)] : 0.f;
    };
    auto request = [&](int base, u32x4_t (&kd)[DA_U], u32x4_t (&vd)[DA_U], float (&md)[DA_U]) {
        __builtin_amdgcn_sched_barrier(0);
        load_rows(kbase, knrow, base, kd);
        load_rows(vbase, vnrow, base, vd);
        load_mask(base, md);
        __builtin_amdgcn_sched_barrier(0);  // the requests go out here, ahead of the arithmetic that follows
    };
    auto consume = [&](int base, const u32x4_t (&kcur)[DA_U], const u32x4_t (&vcur)[DA_U], const float (&mcur)[DA_U]) {
        float sc[DA_U];
        float mx = m;
#pragma unroll
        for (int u = 0; u < DA_U; u++) {
            const half8_t kv = bit_cast<half8_t>(kcur[u]);
            float s = __builtin_amdgcn_fdot2((half2_t){kv[0], kv[1]}, q01, 0.f, false);
            s = __builtin_amdgcn_fdot2((half2_t){kv[2], kv[3]}, q23, s, false);
            s = __builtin_amdgcn_fdot2((half2_t){kv[4], kv[5]}, q45, s, false);
            s = __builtin_amdgcn_fdot2((half2_t){kv[6], kv[7]}, q67, s, false);
            s = quad_sum(s);
            s = xor_sum(s, 4);
            if (LPR == 16) s = xor_sum(s, 8);
            const int j = base + u * RPI + r;
            s = s * a.scale + mcur[u];
            sc[u] = j < r1 ? s : -INFINITY;
            mx = fmaxf(mx, sc[u]);
        }
        // exp(-inf - -inf) is kept out: a slot that has seen only masked rows stays at (m, l) = (-inf, 0)
        const float rescale = (m == -INFINITY) ? 0.f : __expf(m - mx);
        l *= rescale;
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] *= rescale;
#pragma unroll
        for (int u = 0; u < DA_U; u++) {
            const float p = (sc[u] == -INFINITY) ? 0.f : __expf(sc[u] - mx);
            l += p;
            const half8_t vv = bit_cast<half8_t>(vcur[u]);
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] += p * (float)vv[i];
        }
        m = mx;
    };
    // Two register sets take turns (a loop that copied "next" into "current" would have to wait for the
    // requests it has just made); two batches per trip while two are left, then the odd one (a trip's last
    // request may lie past the end of the share: it re-reads the last row and nobody consumes it).
    int base = r0 + wave * RPI * DA_U;
    if (base < r1) {
        request(base, ka, va, ma);
        while (base + STEP < r1) {
            request(base + STEP, kb, vb, mb_);
            consume(base, ka, va, ma);
            request(base + 2 * STEP, ka, va, ma);
            consume(base + STEP, kb, vb, mb_);
            base += 2 * STEP;
        }
        if (base < r1) consume(base, ka, va, ma);
    }

    // Merge the row slots of a wave (lanes with equal c), then the waves.
    float mw = m;
#pragma unroll
    for (int x = LPR; x < 64; x <<= 1) mw = fmaxf(mw, __shfl_xor(mw, x, 64));
    const float sw = (m == -INFINITY) ? 0.f : __expf(m - mw);
    l *= sw;
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] *= sw;
#pragma unroll
    for (int x = LPR; x < 64; x <<= 1) {
        l = xor_sum(l, x);
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = xor_sum(acc[i], x);
    }
    if (lane == 0) {
        mred[wave] = mw;
        lred[wave] = l;
    }
    if (r == 0) {
#pragma unroll
        for (int i = 0; i < 8; i++) ored[wave][8 * c + i] = acc[i];
    }
    __syncthreads();
    float mb = mred[0];
#pragma unroll
    for (int w = 1; w < DA_WAVES; w++) mb = fmaxf(mb, mred[w]);
    float lsum = 0.f, o = 0.f;
    if (tid < D) {
#pragma unroll
        for (int w = 0; w < DA_WAVES; w++) {
            const float f = (mred[w] == -INFINITY) ? 0.f : __expf(mred[w] - mb);
            lsum += lred[w] * f;
            o += ored[w][tid] * f;
        }
    }
    if (nsplit == 1) {
        if (tid < D) a.o[(long)blockIdx.x * D + tid] = (half_t)(o / lsum);  // nothing visible: 0 / 0 = NaN, as the reference
        return;
    }
    // Partial state of this share: [m, l, o[0..D)], exchanged at the device-coherent level (relaxed
    // agent-scope accesses, ordered by the wait below and the counter; no device-wide fence).
    float* mine = a.part + ((long)blockIdx.x * nsplit + blockIdx.y) * (D + 2);
    if (tid < D) __hip_atomic_store(mine + 2 + tid, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) {
        __hip_atomic_store(mine, mb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + 1, lsum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned old = __hip_atomic_fetch_add(&a.counters[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = (old == (unsigned)(nsplit - 1)) ? 1u : 0u;
    }
    __syncthreads();
    if (!last_flag) return;
    if (tid < D) {
        const float* all = a.part + (long)blockIdx.x * nsplit * (D + 2);
        float mg = -INFINITY;
        for (int sp = 0; sp < nsplit; sp++)
            mg = fmaxf(mg, __hip_atomic_load(all + sp * (D + 2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        float lg = 0.f, og = 0.f;
        for (int sp = 0; sp < nsplit; sp++) {  // fixed order: bit-reproducible
            const float ms = __hip_atomic_load(all + sp * (D + 2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const float f = (ms == -INFINITY) ? 0.f : __expf(ms - mg);
            lg += __hip_atomic_load(all + sp * (D + 2) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * f;
            og += __hip_atomic_load(all + sp * (D + 2) + 2 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * f;
        }
        a.o[(long)blockIdx.x * D + tid] = (half_t)(og / lg);
    }
    if (tid == 0) __hip_atomic_store(&a.counters[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int D>
hipError_t launch_d(const DecodeAttnArgs& a, int B, int nsplit, hipStream_t st) {
    if (a.mask)
        hipLaunchKernelGGL((decode_attn_kernel<D, true>), dim3(B * a.H, nsplit), dim3(64 * DA_WAVES), 0, st, a);
    else
        hipLaunchKernelGGL((decode_attn_kernel<D, false>), dim3(B * a.H, nsplit), dim3(64 * DA_WAVES), 0, st, a);
    return hipGetLastError();
}

}  // namespace

// Rows of a head are shared only with fewer than 256 (batch, head) pairs, so 256 counters are
// always enough: the counter region has one fixed size and the partial states one fixed offset,
// whatever B * H a workspace is used with next.
constexpr size_t DECODE_ATTN_COUNTER_BYTES = 256 * sizeof(unsigned);

size_t decode_attention_workspace_bytes(int B, int H, int D) {
    return DECODE_ATTN_COUNTER_BYTES + (size_t)B * H * DECODE_ATTN_MAX_SPLIT * (D + 2) * sizeof(float);
}

hipError_t launch_decode_attention(const void* q, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                                   const void* mask, void* out, int B, int H, int D, int Lmax, long q_bs, long q_hs,
                                   long n_bs, long n_hs, long c_bs, long c_hs, long m_bs, int cache_len,
                                   const long long* cache_len_dev, float sm_scale, void* workspace,
                                   size_t workspace_bytes, hipStream_t st) {
    // Shares per head: enough workgroups for the 256 CUs, at least 128 rows each (what one pass of
    // the eight waves covers), only with a workspace that holds the partial states.
    int nsplit = 1;
    const long heads = (long)B * H;
    if (workspace && heads < 256) {
        const int rows = cache_len_dev ? Lmax : cache_len + (k_new ? 1 : 0);
        while (nsplit < DECODE_ATTN_MAX_SPLIT && heads * nsplit * 2 <= 256 && rows / (nsplit * 2) >= 128) nsplit *= 2;
        if (workspace_bytes < decode_attention_workspace_bytes(B, H, D)) nsplit = 1;
    }
    DecodeAttnArgs a;
    a.q = (const half_t*)q;
    a.kn = (const half_t*)k_new;
    a.vn = (const half_t*)v_new;
    a.kc = (half_t*)k_cache;
    a.vc = (half_t*)v_cache;
    a.mask = (const half_t*)mask;
    a.o = (half_t*)out;
    a.q_bs = q_bs;
    a.q_hs = q_hs;
    a.n_bs = n_bs;
    a.n_hs = n_hs;
    a.c_bs = c_bs;
    a.c_hs = c_hs;
    a.m_bs = m_bs;
    a.H = H;
    a.Lmax = Lmax;
    a.cache_len = cache_len;
    a.cache_len_dev = cache_len_dev;
    a.scale = sm_scale;
    a.counters = (unsigned*)workspace;
    a.part = workspace ? (float*)((char*)workspace + DECODE_ATTN_COUNTER_BYTES) : nullptr;
    return D == 64 ? launch_d<64>(a, B, nsplit, st) : launch_d<128>(a, B, nsplit, st);
}

}  // namespace sq
