/* CPU oracle for the W4A16 linear, plain C.  TEST INFRASTRUCTURE ONLY.
 *
 * Second, independent restatement of the reference algorithm (the first is
 * w4a16_oracle.py); the tests require the two to agree bit for bit on the
 * dequantised weight.  Nothing in the product path links or loads this file.
 *
 * Build: gcc -O2 -fopenmp -shared -fPIC w4a16_oracle.c -o _build/libw4a16_oracle.so
 *
 * Follows, for layout L1 (uint32 [N,K/8], half2 (z+64,s) [N,K/g]):
 *   unpack      quantization/muxi/backend/utils.cuh:81-134
 *   (h-z)*s     quantization/muxi/backend/w4a16_gemm.cuh:58-81
 *   zs index    quantization/muxi/backend/w4a16_gemm.cuh:52  (row*K/g + k/g)
 *   dequant op  quantization/tianshu/backend/w4a16_gemm.cuh:1060-1154
 * fp16 arithmetic is emulated: the difference of two values in [64,79] and the
 * product of two fp16 numbers are exact in binary32, so one final
 * round-to-nearest-even conversion gives the IEEE fp16 result.
 */
#include <stdint.h>
#include <string.h>

static float h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t abs = x & 0x7FFFFFFFu;
    if (abs >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((abs > 0x7F800000u) ? 0x200u : 0));
    if (abs >= 0x477FF000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (abs < 0x38800000u) { /* below the smallest normal half: subnormal */
        if (abs < 0x33000000u) /* < 2^-25 rounds to zero */
            return (uint16_t)sign;
        uint32_t e = abs >> 23;
        uint32_t m = (abs & 0x7FFFFFu) | 0x800000u;
        uint32_t shift = 126u - e; /* bits dropped: 14 .. 24 */
        uint32_t half_m = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_m & 1u)))
            half_m++;
        return (uint16_t)(sign | half_m);
    }
    uint32_t e = (abs >> 23) - 112u;
    uint32_t m = abs & 0x7FFFFFu;
    uint32_t h = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u)))
        h++;
    return (uint16_t)(sign | h);
}

/* uint32 -> 8 fp16 bit patterns of 64 + nibble, in natural k order for L1. */
static void unpack8(uint32_t w, uint16_t out[8]) {
    uint32_t top = w >> 8;
    uint32_t h[4];
    h[0] = ((w & 0x000F000Fu) | 0x05400540u) << 4;
    h[1] = (w & 0x00F000F0u) | 0x54005400u;
    h[2] = ((top & 0x000F000Fu) | 0x05400540u) << 4;
    h[3] = (top & 0x00F000F0u) | 0x54005400u;
    for (int i = 0; i < 4; i++) {
        out[2 * i] = (uint16_t)(h[i] & 0xFFFFu);
        out[2 * i + 1] = (uint16_t)(h[i] >> 16);
    }
}

static uint16_t dq1(uint16_t h, uint16_t z64, uint16_t s) {
    float d = h2f(h) - h2f(z64);      /* exact */
    uint16_t dh = f2h(d);             /* exact, kept for fidelity */
    return f2h(h2f(dh) * h2f(s));     /* one rounding */
}

void sq_oracle_unpack8(uint32_t w, uint16_t* out) { unpack8(w, out); }
uint16_t sq_oracle_f2h(float f) { return f2h(f); }
float sq_oracle_h2f(uint16_t h) { return h2f(h); }

/* W_hat fp16 [N,K] from L1 weight. */
void sq_oracle_dequant_l1(const uint32_t* w, const uint16_t* zs, uint16_t* out,
                          int N, int K, int g) {
    const int groups = K / g;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; n++) {
        for (int k8 = 0; k8 < K / 8; k8++) {
            uint16_t h[8];
            unpack8(w[(size_t)n * (K / 8) + k8], h);
            const uint16_t* p = zs + 2 * ((size_t)n * groups + (k8 * 8) / g);
            for (int i = 0; i < 8; i++)
                out[(size_t)n * K + k8 * 8 + i] = dq1(h[i], p[0], p[1]);
        }
    }
}

/* Y fp32 [M,N] = X fp16 [M,K] * W_hat^T, fp32 accumulate in k order. */
void sq_oracle_gemm_l1(const uint16_t* x, const uint32_t* w, const uint16_t* zs,
                       float* y, int M, int N, int K, int g) {
    const int groups = K / g;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; n++) {
        float wrow[8];
        for (int m = 0; m < M; m++) y[(size_t)m * N + n] = 0.0f;
        for (int k8 = 0; k8 < K / 8; k8++) {
            uint16_t h[8];
            unpack8(w[(size_t)n * (K / 8) + k8], h);
            const uint16_t* p = zs + 2 * ((size_t)n * groups + (k8 * 8) / g);
            for (int i = 0; i < 8; i++) wrow[i] = h2f(dq1(h[i], p[0], p[1]));
            for (int m = 0; m < M; m++) {
                const uint16_t* xr = x + (size_t)m * K + k8 * 8;
                float acc = y[(size_t)m * N + n];
                for (int i = 0; i < 8; i++) acc += h2f(xr[i]) * wrow[i];
                y[(size_t)m * N + n] = acc;
            }
        }
    }
}
