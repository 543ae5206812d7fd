// Shared device helpers for the W4A16 kernels (gfx950 / CDNA4, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sq {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

template <typename To, typename From>
__device__ __forceinline__ To bit_cast(const From& v) {
    static_assert(sizeof(To) == sizeof(From), "size mismatch");
    return __builtin_bit_cast(To, v);
}

// The two nibble masks, pinned in VGPRs: on gfx9-family encodings a VOP3
// instruction takes no literal and at most one scalar operand, so
// (w & mask) | magic becomes a single v_and_or_b32 only with the mask in a VGPR
// and the magic number in an SGPR.
struct NibbleMasks {
    uint32_t lo, hi;
};
__device__ __forceinline__ NibbleMasks nibble_masks() {
    NibbleMasks m = {0x000F000Fu, 0x00F000F0u};
    asm("" : "+v"(m.lo));
    asm("" : "+v"(m.hi));
    return m;
}

// One packed word (layout L1: nibbles k0,k2,k4,k6,k1,k3,k5,k7 from the least
// significant) -> four half2 bit patterns holding 64 + q for (k0,k1), (k2,k3),
// (k4,k5), (k6,k7).  0x5400 is fp16 64.0 and ulp(64) = 1/16, so a nibble placed
// in mantissa bits 4..7 adds exactly its value.
// (reference: quantization/muxi/backend/utils.cuh:81-134)
__device__ __forceinline__ void unpack8_bias64(uint32_t w, uint32_t h[4], const NibbleMasks& nm) {
    const uint32_t t = w >> 8;
    h[0] = ((w & nm.lo) | 0x05400540u) << 4;
    h[1] = (w & nm.hi) | 0x54005400u;
    h[2] = ((t & nm.lo) | 0x05400540u) << 4;
    h[3] = (t & nm.hi) | 0x54005400u;
}

// (h - z64) * s on a half2, each operation rounded once in fp16: the difference
// of two values in [64,79] is exact, so the result is the correctly rounded
// (q - z) * s.  (reference: quantization/muxi/backend/w4a16_gemm.cuh:58-81)
__device__ __forceinline__ uint32_t dequant_pair(uint32_t h, half2_t zb, half2_t s) {
    half2_t v = bit_cast<half2_t>(h);
    v = (v - zb) * s;
    return bit_cast<uint32_t>(v);
}

// Word -> 8 dequantised fp16 (natural k order) as one 128-bit value, bit-identical
// to fp16 (q - z) * s.  Low nibbles are unpacked without a shift as 1024 + q
// (magic 0x6400), high nibbles as 64 + q (magic 0x5400); the stored zero 64 + z is
// used as is for the high ones and as 1024 + z (= stored zero + 960, exact in fp16)
// for the low ones, so both differences are the exact integer q - z.
__device__ __forceinline__ half8_t dequant8(uint32_t w, half2_t z64, half2_t s, const NibbleMasks& nm) {
    const half2_t z1024 = z64 + (half2_t){(half_t)960.f, (half_t)960.f};
    const uint32_t t = w >> 8;
    u32x4_t r;
    r.x = dequant_pair((w & nm.lo) | 0x64006400u, z1024, s);
    r.y = dequant_pair((w & nm.hi) | 0x54005400u, z64, s);
    r.z = dequant_pair((t & nm.lo) | 0x64006400u, z1024, s);
    r.w = dequant_pair((t & nm.hi) | 0x54005400u, z64, s);
    return bit_cast<half8_t>(r);
}

// Word -> 8 fp16 holding 64 + q (no zero / scale applied).
__device__ __forceinline__ half8_t unpack8_raw(uint32_t w, const NibbleMasks& nm) {
    uint32_t h[4];
    unpack8_bias64(w, h, nm);
    u32x4_t r = {h[0], h[1], h[2], h[3]};
    return bit_cast<half8_t>(r);
}

// Sum over the four lanes {l, l^4, l^8, l^12} of a 16-lane row using DPP row
// rotations (no LDS traffic).
__device__ __forceinline__ float row_sum_stride4(float v) {
    int i = bit_cast<int>(v);
    v += bit_cast<float>(__builtin_amdgcn_update_dpp(0, i, 0x124, 0xF, 0xF, false));  // row_ror:4
    i = bit_cast<int>(v);
    v += bit_cast<float>(__builtin_amdgcn_update_dpp(0, i, 0x128, 0xF, 0xF, false));  // row_ror:8
    return v;
}

// Sum over the four lanes of a quad (lanes 4q .. 4q+3), result in every lane.
__device__ __forceinline__ float quad_sum(float v) {
    v += bit_cast<float>(__builtin_amdgcn_update_dpp(0, bit_cast<int>(v), 0xB1, 0xF, 0xF, false));  // quad_perm 1,0,3,2
    v += bit_cast<float>(__builtin_amdgcn_update_dpp(0, bit_cast<int>(v), 0x4E, 0xF, 0xF, false));  // quad_perm 2,3,0,1
    return v;
}

// Broadcast lane T of every quad to the four lanes of that quad (128-bit value).
template <int T>
__device__ __forceinline__ u32x4_t quad_bcast(u32x4_t v) {
    constexpr int ctrl = T * 0x55;  // quad_perm T,T,T,T
    u32x4_t r;
    r.x = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.x, ctrl, 0xF, 0xF, false);
    r.y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.y, ctrl, 0xF, 0xF, false);
    r.z = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.z, ctrl, 0xF, 0xF, false);
    r.w = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.w, ctrl, 0xF, 0xF, false);
    return r;
}

// Word -> 8 fp16 with mixed bias and no shift: 1024 + q at positions 0, 1, 4, 5 (the low nibbles
// land in mantissa bits 0..3 of 0x6400 = 1024, where ulp = 1) and 64 + q at positions 2, 3, 6, 7.
// Five operations instead of seven; the consumer removes the extra 960 on the low positions.
__device__ __forceinline__ half8_t unpack8_mixed(uint32_t w, const NibbleMasks& nm) {
    const uint32_t t = w >> 8;
    u32x4_t r = {(w & nm.lo) | 0x64006400u, (w & nm.hi) | 0x54005400u, (t & nm.lo) | 0x64006400u,
                 (t & nm.hi) | 0x54005400u};
    return bit_cast<half8_t>(r);
}

__device__ __forceinline__ int imin(int a, int b) { return a < b ? a : b; }

// LayerNorm applied to the activations on their way into a linear (fp32 statistics over the K columns of a
// token, biased variance, one rounding to fp16): x_hat = (x - mean) * rsqrt(var + eps) * gamma + beta.
struct LnPre {
    const half_t* gamma;  // [K] or null (1)
    const half_t* beta;   // [K] or null (0)
    float eps;
};

// What happens to an fp32 accumulator on its way to Y[m, n]: + bias[n], activation,
// * mul[m, n], + residual[m, n] (each optional), one rounding to fp16 at the end.
struct Epilogue {
    const half_t* bias;      // [N] or null
    const half_t* residual;  // [M, N] or null; must not overlap Y
    int act;                 // 0 = none, 1 = ReLU, 2 = SiLU
    const half_t* mul = nullptr;  // [M, N] or null; must not overlap Y (the other half of a gated MLP)
};
// The full tail with the multiplicand already in a register (1 where there is none).
__device__ __forceinline__ half_t epilogue_times(float v, float mulv, int m, int n, int N, const Epilogue& e) {
    if (e.bias) v += (float)e.bias[n];
    if (e.act == 1)
        v = fmaxf(v, 0.f);
    else if (e.act == 2)
        v = v * __builtin_amdgcn_rcpf(1.f + __expf(-v));  // v * sigmoid(v); exp overflows to +inf for v << 0, the product is -0
    v *= mulv;
    if (e.residual) v += (float)e.residual[(long)m * N + n];
    return (half_t)v;
}
__device__ __forceinline__ half_t epilogue(float v, int m, int n, int N, const Epilogue& e) {
    return epilogue_times(v, e.mul ? (float)e.mul[(long)m * N + n] : 1.f, m, n, N, e);
}

// Four consecutive outputs of one row (n a multiple of 4; N is a multiple of 8, so they are inside or outside
// together) whose bias and residual are requested ahead of the data they meet: the last workgroup of a K split
// asks for them before it fetches the partial tiles, so that the two round trips overlap.
struct Tail4 {
    u32x2_t bias, res;
};
__device__ __forceinline__ bool tail4_applies(const Epilogue& e) {
    return e.mul == nullptr && (reinterpret_cast<uintptr_t>(e.bias) & 7u) == 0 &&
           (reinterpret_cast<uintptr_t>(e.residual) & 7u) == 0;
}
__device__ __forceinline__ Tail4 tail4_request(const Epilogue& e, int m, int n, int N, bool inside) {
    Tail4 t = {{0u, 0u}, {0u, 0u}};
    if (e.bias && inside) t.bias = *(const u32x2_t*)(e.bias + n);
    if (e.residual && inside) t.res = *(const u32x2_t*)(e.residual + (long)m * N + n);
    return t;
}
__device__ __forceinline__ void tail4_store(float4_t v, const Tail4& t, half_t* __restrict__ Y, int m, int n, int N,
                                            const Epilogue& e) {
    const half4_t b = bit_cast<half4_t>(t.bias), r = bit_cast<half4_t>(t.res);
    half4_t o;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float x = v[i];
        if (e.bias) x += (float)b[i];
        if (e.act == 1)
            x = fmaxf(x, 0.f);
        else if (e.act == 2)
            x = x * __builtin_amdgcn_rcpf(1.f + __expf(-x));
        if (e.residual) x += (float)r[i];
        o[i] = (half_t)x;
    }
    *(half4_t*)(Y + (long)m * N + n) = o;
}

// Eight consecutive fp16 values as floats: one 128-bit load where the pointer allows it.
__device__ __forceinline__ void load8_halves(const half_t* p, bool aligned, float (&out)[8]) {
    if (aligned) {
        const half8_t h = *(const half8_t*)p;
#pragma unroll
        for (int e = 0; e < 8; e++) out[e] = (float)h[e];
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) out[e] = (float)p[e];
    }
}

// The tail of the tiled GEMM kernels: a workgroup of four waves holds a (32 MI) x 256 tile of fp32 sums in the
// matrix instruction's layout (wave w: columns 64 w .. +63; acc[mi][ni][v] of lane (ln, lc) = row
// 32 mi + 8 (v / 4) + 4 lc + v % 4, column 32 ni + ln).  Stored straight from that layout every lane would issue
// one 2-byte access per element, and the memory pipeline takes those one lane at a time (128 of them per lane
// for a 128-row tile, and as many again for each of bias, multiplicand and residual).  Instead each 32-row
// slice goes through LDS as fp32 and comes back row-major, eight consecutive columns per thread: bias,
// activation, multiplicand, residual and the one rounding to fp16 happen there, and every global access of the
// tail is 128 bits wide with neighbouring lanes on neighbouring addresses.  Same operations in the same order as
// epilogue(): bit-identical results.  lds: 32 KiB of the workgroup's shared memory that nothing else uses any
// more (the first barrier below separates it from the main loop's reads).
template <int MI>
__device__ __forceinline__ void tile_store_via_lds(const float16_t (&acc)[MI][2], half_t* __restrict__ Y, int M, int N,
                                                   int m0, int nb, const Epilogue& epi, float* lds) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int ln = lane & 31;
    const int lc = lane >> 5;
    const int c8 = tid & 31;  // this thread's chunk of eight columns on the way out
    const int r0 = tid >> 5;  // and its first row; the others follow in steps of 8
    const int n = nb + 8 * c8;
    const bool col_ok = n < N;  // N is a multiple of 8: a chunk is inside or outside as a whole
    float bias8[8];
#pragma unroll
    for (int e = 0; e < 8; e++) bias8[e] = 0.f;
    if (epi.bias && col_ok) load8_halves(epi.bias + n, (reinterpret_cast<uintptr_t>(epi.bias) & 15u) == 0, bias8);
    const bool res_aligned = (reinterpret_cast<uintptr_t>(epi.residual) & 15u) == 0;
    const bool mul_aligned = (reinterpret_cast<uintptr_t>(epi.mul) & 15u) == 0;
#pragma unroll
    for (int mi = 0; mi < MI; mi++) {
        __syncthreads();
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                lds[(8 * (v >> 2) + 4 * lc + (v & 3)) * 256 + 64 * wave + 32 * ni + ln] = acc[mi][ni][v];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int r = r0 + 8 * j;
            const int m = m0 + 32 * mi + r;
            if (m < M && col_ok) {
                const float4_t lo = *(const float4_t*)(lds + r * 256 + 8 * c8);
                const float4_t hi = *(const float4_t*)(lds + r * 256 + 8 * c8 + 4);
                float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                const long idx = (long)m * N + n;
                if (epi.bias) {
#pragma unroll
                    for (int e = 0; e < 8; e++) v[e] += bias8[e];
                }
                if (epi.act == 1) {
#pragma unroll
                    for (int e = 0; e < 8; e++) v[e] = fmaxf(v[e], 0.f);
                } else if (epi.act == 2) {
#pragma unroll
                    for (int e = 0; e < 8; e++) v[e] = v[e] * __builtin_amdgcn_rcpf(1.f + __expf(-v[e]));
                }
                if (epi.mul) {
                    float t[8];
                    load8_halves(epi.mul + idx, mul_aligned, t);
#pragma unroll
                    for (int e = 0; e < 8; e++) v[e] *= t[e];
                }
                if (epi.residual) {
                    float t[8];
                    load8_halves(epi.residual + idx, res_aligned, t);
#pragma unroll
                    for (int e = 0; e < 8; e++) v[e] += t[e];
                }
                half8_t h;
#pragma unroll
                for (int e = 0; e < 8; e++) h[e] = (half_t)v[e];
                *(half8_t*)(Y + idx) = h;
            }
        }
    }
}

// 128-bit global accesses at the device-coherent level (cache policy sc1, what agent-scope
// relaxed atomics use), for data exchanged between workgroups inside one kernel.  The eight
// loads and the wait for them are one asm statement, so the compiler never sees a register
// whose data is still in flight.
__device__ __forceinline__ void store_coherent_x4(float* p, float4_t v) {
    // The trailing s_nop covers the hazard between a wide store and a later overwrite of its
    // data registers, which the compiler cannot see through inline asm.
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 3" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void load8_coherent_x4(const float* const (&p)[8], float4_t (&v)[8]) {
    asm volatile(
        "global_load_dwordx4 %0, %8, off sc1\n\t"
        "global_load_dwordx4 %1, %9, off sc1\n\t"
        "global_load_dwordx4 %2, %10, off sc1\n\t"
        "global_load_dwordx4 %3, %11, off sc1\n\t"
        "global_load_dwordx4 %4, %12, off sc1\n\t"
        "global_load_dwordx4 %5, %13, off sc1\n\t"
        "global_load_dwordx4 %6, %14, off sc1\n\t"
        "global_load_dwordx4 %7, %15, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7])
        : "memory");
}

// One direct global -> LDS load: 16 (or 4) bytes per lane, lane l lands at lds_byte + 16 (4) * l.
// Written as inline assembly on purpose: the compiler, when it knows of such a load, makes every
// later LDS read wait for ALL outstanding vector memory loads unless it can prove the two apart,
// which it cannot for stages picked at run time.  The kernel orders them itself (a counted
// s_waitcnt and a barrier per step); the "memory" clobbers keep LDS reads from moving across.
// The LDS address travels in m0, bound as an input so that the compiler knows the register is written.
__device__ __forceinline__ void load_to_lds_x4(const void* g, uint32_t lds_byte) {
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "{m0}"(lds_byte) : "memory");
}
__device__ __forceinline__ void load_to_lds_x1(const void* g, uint32_t lds_byte) {
    asm volatile("s_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(g), "{m0}"(lds_byte) : "memory");
}
// The same with the address split into a wave-uniform base and a 32-bit byte offset per lane: a loop that
// walks along K then advances one scalar instead of one 64-bit sum per lane and load.
__device__ __forceinline__ void load_to_lds_x4(const void* base, uint32_t lane_byte, uint32_t lds_byte) {
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_byte), "s"(base), "{m0}"(lds_byte) : "memory");
}
__device__ __forceinline__ void load_to_lds_x1(const void* base, uint32_t lane_byte, uint32_t lds_byte) {
    asm volatile("s_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(lane_byte), "s"(base), "{m0}"(lds_byte) : "memory");
}

// Sixteen coherent 128-bit loads in flight: p[i] points at the SECOND of two locations 4096 bytes
// apart (v[2i] = p[i][-4096 bytes], v[2i+1] = p[i][0]); one asm block with its own wait, so that no
// register holding a result can be touched before the data is there.
__device__ __forceinline__ void load16_coherent_x4(const float* const (&p)[8], float4_t (&v)[16]) {
    asm volatile(
        "global_load_dwordx4 %0, %16, off offset:-4096 sc1\n\t"
        "global_load_dwordx4 %1, %16, off sc1\n\t"
        "global_load_dwordx4 %2, %17, off offset:-4096 sc1\n\t"
        "global_load_dwordx4 %3, %17, off sc1\n\t"
        "global_load_dwordx4 %4, %18, off offset:-4096 sc1\n\t"
        "global_load_dwordx4 %5, %18, off sc1\n\t"
        "global_load_dwordx4 %6, %19, off offset:-4096 sc1\n\t"
        "global_load_dwordx4 %7, %19, off sc1\n\t"
        "global_load_dwordx4 %8, %20, off offset:-4096 sc1\n\t"
        "global_load_dwordx4 %9, %20, off sc1\n\t"
        "global_load_dwordx4 %10, %21, off offset:-4096 sc1\n\t"
        "global_load_dwordx4 %11, %21, off sc1\n\t"
        "global_load_dwordx4 %12, %22, off offset:-4096 sc1\n\t"
        "global_load_dwordx4 %13, %22, off sc1\n\t"
        "global_load_dwordx4 %14, %23, off offset:-4096 sc1\n\t"
        "global_load_dwordx4 %15, %23, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7]),
          "=&v"(v[8]), "=&v"(v[9]), "=&v"(v[10]), "=&v"(v[11]), "=&v"(v[12]), "=&v"(v[13]), "=&v"(v[14]), "=&v"(v[15])
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7])
        : "memory");
}

}  // namespace sq
