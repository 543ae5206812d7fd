// C ABI of libsq_w4a16.so: argument validation and kernel dispatch.  Declarations
// and the contract of every entry point are in include/sq_w4a16.h.
#include "../../include/sq_w4a16.h"

#include <atomic>
#include <mutex>

#include "sq_kernels.h"

// Workspace of sq_w4a16_gemm_static_ws: device memory that belongs to the library, so that the
// call allocates nothing.  Every GPU the library runs on holds its own copy of the array until the
// process ends; the name below is only the host-side handle of the symbol, the device address is
// looked up once per device with hipGetSymbolAddress and that pointer is what the kernels get.
static __device__ __align__(256) unsigned char scratch[SQ_STATIC_WS_BYTES];

namespace {

__global__ void zero_words_kernel(unsigned* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

constexpr int MAX_DEVICES = 64;
void* g_scratch[MAX_DEVICES];
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (null on failure).  The array needs no clearing: a
// file-scope __device__ array without an initialiser is zero when its code object is loaded, and every kernel
// leaves the counters at its start zero.
void* static_workspace() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
        g_scratch[dev] = p;
    }
    return g_scratch[dev];
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int launch_code(hipError_t e) { return e == hipSuccess ? SQ_OK : SQ_ERR_LAUNCH; }
inline bool pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

// Shape rules shared by gemm and dequant.
int check_weight(int N, int K, int g, int layout) {
    if (layout != SQ_LAYOUT_L1 && layout != SQ_LAYOUT_L2) return SQ_ERR_BAD_LAYOUT;
    if (N <= 0 || K <= 0) return SQ_ERR_BAD_SHAPE;
    if (layout == SQ_LAYOUT_L1) {
        if (g != 32 && g != 64 && g != 128) return SQ_ERR_BAD_GROUP;
        if (N % 8 != 0 || K % 32 != 0 || K % g != 0) return SQ_ERR_BAD_SHAPE;
    } else {
        if (g != 128) return SQ_ERR_BAD_GROUP;
        if (N % 32 != 0 || K % 32 != 0 || K % g != 0) return SQ_ERR_BAD_SHAPE;
    }
    if ((long)N * (long)K > (1L << 40)) return SQ_ERR_BAD_SHAPE;
    return SQ_OK;
}

// One dispatcher behind every GEMM entry point.  `workspace` may be null: then the kernels
// that need one are not considered (and an explicit SQ_ALGO_SKINNY_WS is an error).
// Measured kernel choices (sq_w4a16_autotune): shape -> kernel word, consulted before the built-in rules.
// Entries are only ever appended (under the mutex); readers scan without it up to the published count.
struct TunedEntry {
    int M, N, K, g, has_ws, algo;
    float us;
};
constexpr int TUNED_MAX = 1024;
TunedEntry g_tuned[TUNED_MAX];
std::atomic<int> g_tuned_count{0};
std::mutex g_tuned_mutex;

inline bool full_workspace(const void* workspace, size_t workspace_bytes, int M, int N, int K) {
    return workspace && (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0 &&
           workspace_bytes >= sq_w4a16_workspace_bytes(M, N, K);
}

int tuned_lookup(int M, int N, int K, int g, bool has_ws) {
    const int n = g_tuned_count.load(std::memory_order_acquire);
    for (int i = n - 1; i >= 0; i--) {  // the latest measurement of a shape wins
        const TunedEntry& e = g_tuned[i];
        if (e.M == M && e.N == N && e.K == K && e.g == g && e.has_ws == (int)has_ws) return e.algo;
    }
    return 0;
}

// The built-in kernel choice as a table: the first row whose token range contains M, whose `need` properties all
// hold and whose `forbid` properties all fail names the kernel.  Every row carries the measurement it rests on
// (MI355X, cold weights, OPT-6.7B / Llama-2-7B shapes, us per launch).  sq_w4a16_autotune overrides the table per
// shape with a measurement of that shape.
enum : unsigned {
    P_LARGE = 1u << 0,      // N * K >= 2^25 elements (fc1 / fc2 class)
    P_WS = 1u << 1,         // a workspace for the decode kernels' K split is at hand
    P_GEMM_WS = 1u << 2,    // a workspace for the tiled GEMM's K split is at hand
    P_G128 = 1u << 3,       // group size 128
    P_G128_64 = 1u << 4,    // group size 128 or 64
    P_K128 = 1u << 5,       // K a multiple of 128
    P_K256 = 1u << 6,       // K a multiple of 256
    P_K_LE_4096 = 1u << 7,
    P_K_LE_8192 = 1u << 8,
    P_K_LE_32768 = 1u << 9,
    P_WIDE = 1u << 10,      // the two-tile streaming kernel applies and its workgroups come in one round or fill their rounds
    P_SMALL = 1u << 11,     // N * K <= 2^22 elements and K <= 2048
    P_N_GE_8192 = 1u << 12, // 32 or more 256-column tiles: a K split of up to 8 gives every CU a workgroup of the tiled GEMM
    P_K_LE_1536 = 1u << 13,
    P_CHUNK_FILL = 1u << 14,  // the least K split of the streaming kernel fills 3/4 or more of a workgroup's 32 chunks
};
constexpr int ALGO_TWO_BLOCKS = 100;  // internal: the split-K decode kernel on two blocks of up to 32 tokens
struct ChoiceRule {
    int m_lo, m_hi;
    unsigned need, forbid;
    int kernel;
    const char* measured;
};
const ChoiceRule kChoiceRules[] = {
    // the streaming decode kernel, 5..16 tokens (3..4 on large weights); K beyond 4096 is split through the workspace
    {5, 16, P_G128_64 | P_K128 | P_K_LE_4096, 0, SQ_ALGO_STREAM,
     "8 tokens: fc1 10.0 vs 13.3 (split-K kernel), q/k/v in one launch 8.6 vs 12.1, 4096x4096 4.9 vs 6.5 (GEMV)"},
    {5, 16, P_G128_64 | P_K128 | P_WS | P_K_LE_32768, 0, SQ_ALGO_STREAM, "8 tokens: fc2 12.7 vs 14.6 (split-K kernel)"},
    {3, 4, P_LARGE | P_G128_64 | P_K128 | P_K_LE_4096, 0, SQ_ALGO_STREAM, "4 tokens: fc1 9.7 vs 10.7 (GEMV)"},
    {3, 4, P_LARGE | P_G128_64 | P_K128 | P_WS | P_K_LE_32768 | P_CHUNK_FILL, 0, SQ_ALGO_STREAM,
     "4 tokens: fc2 11.9 vs 13.6 (GEMV); 13824x5120, whose K ranges fill 20 of a workgroup's 32 chunks: 14.6 vs 13.9 (GEMV)"},
    // small weights at 17..32 tokens: the 16-column kernel (one launch, no exchange between workgroups)
    {17, 32, P_SMALL, 0, SQ_ALGO_SKINNY,
     "32 tokens: 2048x2048 7.4 vs 8.6 (split-K kernel), 1024x1024 4.9 vs 6.9, 3072x768 4.8 vs 6.6"},
    // its two-tile variant, 17..32 tokens
    {17, 32, P_G128 | P_WIDE, 0, SQ_ALGO_STREAM,
     "32 tokens: fc1 16.5 vs 17.2 (split-K kernel), q/k/v-sized 14.3 vs 15.5, fc2 18.1 vs 19.0"},
    // large weights whose grid leaves the two-tile kernel's last round part empty or whose K leaves chunk slots of
    // its workgroups unused: the tiled GEMM's 32-row tiles with K split through the workspace
    {17, 32, P_LARGE | P_K256 | P_GEMM_WS | P_G128, 0, SQ_ALGO_GEMM,
     "32 tokens: 13824x5120 20.2 vs 27.7 (two-tile kernel: 1.7 rounds of workgroups at 20 of 32 chunk slots), "
     "28672x8192 47.2 vs 56.7, 8192x28672 45.6 vs 55.6, 5120x13824 23.3 vs 26.9, 22016x4096 24.3 vs 25.9"},
    // the same at group size 64 and 32 (no two-tile kernel) on weights with enough columns of tiles; long K on few
    // rows stays with the split-K kernel below (group size 64, 4096x16384: 19.6 vs 25.2 for the tiled GEMM)
    {17, 32, P_LARGE | P_K256 | P_GEMM_WS | P_N_GE_8192, 0, SQ_ALGO_GEMM,
     "32 tokens, group size 64: fc1 18.4, 12288x4096 16.0, 13824x5120 20.7, 28672x8192 53.6: no other kernel faster"},
    // small weights with a short K at 33..64 tokens: still the 16-column kernel (from K = 2048 on the GEMM wins)
    {33, 64, P_SMALL | P_K_LE_1536, 0, SQ_ALGO_SKINNY,
     "48 tokens: 3072x768 5.6 vs 8.6 (tiled GEMM), 4096x1024 6.3 vs 8.6, 1024x1024 5.9 vs 8.1, 1536x1536 7.8 vs 9.9; "
     "64 tokens: 6.8 vs 8.6, 7.3 vs 8.7, 6.9 vs 8.1, 9.2 vs 10.0; 2048x2048 at 64 tokens 12.0 vs 10.7"},
    // the tiled GEMM with every operand through LDS and K split through the workspace, beyond 32 tokens
    {33, 1 << 30, P_K256 | P_GEMM_WS, 0, SQ_ALGO_GEMM,
     "48 tokens: 4096x4096 14.5 vs 17.2 (two blocks of the split-K kernel), fc1 24.7 vs 28.2, fc2 27.0 vs 32.3; "
     "64 tokens: 14.5 vs 20.5 (16-column kernel)"},
    // the split-K decode kernel: where the streaming kernels do not apply (group size 32, K no multiple of 128,
    // grids that leave the two-tile kernel under half the chip such as 4096x4096 at 17..32 tokens)
    {5, 32, P_WS | P_LARGE, 0, SQ_ALGO_SKINNY_WS, "16 tokens: fc1 12.5, fc2 14.7 vs 16-column kernel 19.6 / 21.7"},
    {17, 32, P_WS, 0, SQ_ALGO_SKINNY_WS, "32 tokens: 4096x4096 9.8 vs 10.2 (two-tile kernel at 64 rows x 2048 columns)"},
    {5, 32, P_WS, P_K_LE_8192, SQ_ALGO_SKINNY_WS, "long K: one workgroup per 16 rows cannot stage the activations in one round"},
    {33, 48, P_WS | P_LARGE, 0, ALGO_TWO_BLOCKS, "33..48 tokens without the GEMM's workspace: fc1 30 vs 31 (tiled GEMM), fc2 35 vs 37"},
    {33, 48, P_WS, P_K_LE_8192, ALGO_TWO_BLOCKS, "as above, long K"},
    // the decode GEMV: up to 4 tokens, up to 8 while its staged activations fit one round
    {1, 4, 0, 0, SQ_ALGO_GEMV_FIXUP, "1 token: the four-launch layer step 27.3 per step; 4096x4096 at 4 tokens 4.4"},
    {5, 8, P_K_LE_8192, 0, SQ_ALGO_GEMV_FIXUP, "8 tokens at group size 32 (no streaming kernel): 6.5 vs 8.1 (16-column kernel)"},
    // the 16-column kernel: no workspace, or small weights at 33..64 tokens
    {5, 32, 0, 0, SQ_ALGO_SKINNY, "no workspace: the only kernel of this range that needs none"},
    {33, 64, P_K_LE_8192, P_LARGE, SQ_ALGO_SKINNY, "4096x4096 at 64 tokens without the GEMM's workspace: 21 vs 46 (unsplit GEMM)"},
    {33, 64, 0, P_GEMM_WS | P_K_LE_8192, SQ_ALGO_SKINNY, "4096x16384 at 64 tokens without a workspace: 70 vs 170 (unsplit GEMM)"},
    {1, 1 << 30, 0, 0, SQ_ALGO_GEMM, "everything else: the tiled GEMM (plan_gemm picks tile height, staging and split)"},
};

int builtin_choice(int M, int N, int K, int g, bool ws_ok, bool gemm_ws) {
    unsigned p = 0;
    if ((long)N * (long)K >= (1L << 25)) p |= P_LARGE;
    if (ws_ok) p |= P_WS;
    if (gemm_ws) p |= P_GEMM_WS;
    if (g == 128) p |= P_G128;
    if (g == 128 || g == 64) p |= P_G128_64;
    if (K % 128 == 0) p |= P_K128;
    if (K % 256 == 0) p |= P_K256;
    if ((long)N * (long)K <= (1L << 22) && K <= 2048) p |= P_SMALL;
    if (N >= 8192) p |= P_N_GE_8192;
    if (K <= 1536) p |= P_K_LE_1536;
    {
        const int chunks = K / 128, ks0 = (chunks + 31) / 32;
        if (ks0 > 0 && chunks * 4 >= ks0 * 32 * 3) p |= P_CHUNK_FILL;
    }
    if (K <= 4096) p |= P_K_LE_4096;
    if (K <= 8192) p |= P_K_LE_8192;
    if (K <= 32768) p |= P_K_LE_32768;
    if (M > 16 && M <= 32 && g == 128) {
        // One workgroup per CU: W workgroups take ceil(W / 256) rounds of about the same length whatever part of
        // their 32 chunk slots the K range fills.
        long wgs = 0;
        int slots = 0;
        if (sq::skinny3_wide_shape(N, K, ws_ok, &wgs, &slots)) {
            const long rounds = (wgs + 255) / 256;
            if (wgs <= 256 || wgs * slots * 100 >= rounds * 256 * 32 * 95) p |= P_WIDE;
        }
    }
    for (const ChoiceRule& r : kChoiceRules)
        if (M >= r.m_lo && M <= r.m_hi && (p & r.need) == r.need && (p & r.forbid) == 0) return r.kernel;
    return SQ_ALGO_GEMM;
}

int gemm_dispatch(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int group_size,
                  int layout, int algo, sq::Epilogue epi, void* workspace, size_t workspace_bytes, void* stream) {
    if (M < 0) return SQ_ERR_BAD_SHAPE;
    const int rc = check_weight(N, K, group_size, layout);
    if (rc != SQ_OK) return rc;
    // The GEMM kernels consume layout L1; an L2 weight is converted once with
    // sq_repack_l2_to_l1 by the caller (the `quant` extension caches the result).
    if (layout != SQ_LAYOUT_L1) return SQ_ERR_BAD_LAYOUT;
    if (M == 0) return SQ_OK;
    if (!x || !w || !zs || !y) return SQ_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(w) || !aligned16(zs) || !aligned16(y)) return SQ_ERR_MISALIGNED;
    if ((long)M * (long)K > (1L << 40) || (long)M * (long)N > (1L << 40)) return SQ_ERR_BAD_SHAPE;
    hipStream_t st = static_cast<hipStream_t>(stream);

    int kernel = algo & 0xFF;
    int tune = (algo >> 8) & 0xFFFF;
    if (kernel == SQ_ALGO_AUTO && g_tuned_count.load(std::memory_order_relaxed) > 0) {
        const int word = tuned_lookup(M, N, K, group_size, full_workspace(workspace, workspace_bytes, M, N, K));
        if (word != 0) {
            kernel = word & 0xFF;
            tune = (word >> 8) & 0xFFFF;
        }
    }
    if (kernel == SQ_ALGO_AUTO) {
        const bool ws_ok = workspace && aligned16(workspace) &&
                           workspace_bytes >= sq::skinny2_workspace_bytes(M > 32 ? 32 : M, N, K) &&
                           (N + 63) / 64 <= 16384;
        const bool gemm_ws = workspace && aligned16(workspace) && M > 16 &&
                             workspace_bytes >= sq::gemm_workspace_bytes(M, N, K);
        kernel = builtin_choice(M, N, K, group_size, ws_ok, gemm_ws);
        if (kernel == ALGO_TWO_BLOCKS) {
            for (int m0 = 0; m0 < M; m0 += 32) {
                const int mb = M - m0 < 32 ? M - m0 : 32;
                sq::Epilogue e = epi;
                if (e.residual) e.residual += (long)m0 * N;
                if (e.mul) e.mul += (long)m0 * N;
                const hipError_t err = sq::launch_skinny2_tuned(
                    static_cast<const sq::half_t*>(x) + (long)m0 * K, w, zs, static_cast<sq::half_t*>(y) + (long)m0 * N,
                    workspace, mb, N, K, group_size, 0, e, st);
                if (err != hipSuccess) return SQ_ERR_LAUNCH;
            }
            return SQ_OK;
        }
    }
    switch (kernel) {
        case SQ_ALGO_GEMV:
        case SQ_ALGO_GEMV_FIXUP:
            if (M > 8) return SQ_ERR_BAD_ALGO;
            return launch_code(sq::launch_gemv2_tuned(x, w, zs, y, M, N, K, group_size,
                                                      kernel == SQ_ALGO_GEMV_FIXUP, tune, epi, st));
        case SQ_ALGO_SKINNY:
            if (M > 64) return SQ_ERR_BAD_ALGO;
            return launch_code(sq::launch_skinny_tuned(x, w, zs, y, M, N, K, group_size, tune, epi, st));
        case SQ_ALGO_SKINNY_WS:
            if (M > 32) return SQ_ERR_BAD_ALGO;
            if (!workspace || !aligned16(workspace) || workspace_bytes < sq::skinny2_workspace_bytes(M, N, K) ||
                (N + 63) / 64 > 16384)
                return SQ_ERR_WORKSPACE;
            return launch_code(sq::launch_skinny2_tuned(x, w, zs, y, workspace, M, N, K, group_size, tune, epi, st));
        case SQ_ALGO_STREAM: {
            if (M > 16 && M <= 32 && group_size == 128) {
                const bool ws_fits = workspace && aligned16(workspace) &&
                                     workspace_bytes >= sq::skinny2_workspace_bytes(M, N, K);
                const hipError_t e = sq::launch_skinny3_wide(x, w, zs, y, ws_fits ? workspace : nullptr, M, N, K, epi, st);
                return e == hipErrorInvalidValue ? SQ_ERR_WORKSPACE : launch_code(e);
            }
            if (M > 16 || (group_size != 128 && group_size != 64)) return SQ_ERR_BAD_ALGO;
            const bool ws_fits = workspace && aligned16(workspace) &&
                                 workspace_bytes >= sq::skinny2_workspace_bytes(M, N, K);
            const hipError_t e =
                sq::launch_skinny3_tuned(x, w, zs, y, ws_fits ? workspace : nullptr, M, N, K, group_size, tune, epi, nullptr, st);
            return e == hipErrorInvalidValue ? SQ_ERR_WORKSPACE : launch_code(e);
        }
        case SQ_ALGO_GEMM:
            return launch_code(sq::launch_gemm_tuned(x, w, zs, y, aligned16(workspace) ? workspace : nullptr,
                                                     workspace_bytes, M, N, K, group_size, tune, epi, st));
        default:
            return SQ_ERR_BAD_ALGO;
    }
}

}  // namespace

extern "C" {

int sq_version(void) { return 100; }

const char* sq_strerror(int code) {
    switch (code) {
        case SQ_OK: return "ok";
        case SQ_ERR_NULL_POINTER: return "null pointer argument";
        case SQ_ERR_BAD_SHAPE: return "unsupported shape (need N % 8 == 0, K % 32 == 0, K % group_size == 0)";
        case SQ_ERR_BAD_GROUP: return "unsupported group size";
        case SQ_ERR_BAD_LAYOUT: return "unknown or unsupported weight layout";
        case SQ_ERR_BAD_ALGO: return "unknown kernel id or kernel not applicable to this shape";
        case SQ_ERR_MISALIGNED: return "pointer is not 16-byte aligned";
        case SQ_ERR_LAUNCH: return "HIP kernel launch failed";
        case SQ_ERR_WORKSPACE: return "workspace missing or too small";
        case SQ_ERR_STATIC_WS: return "problem needs a larger workspace than the library's static buffer (SQ_STATIC_WS_BYTES)";
        case SQ_ERR_SEQ_TIMEOUT: return "a one-launch sequence gave up waiting for another workgroup's output (results of that call are undefined)";
        default: return "unknown error code";
    }
}

int sq_w4a16_gemm_ex(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int group_size,
                     int layout, int algo, void* stream) {
    return gemm_dispatch(x, w, zs, y, M, N, K, group_size, layout, algo, sq::Epilogue{nullptr, nullptr, 0}, nullptr, 0,
                         stream);
}

size_t sq_w4a16_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const size_t a = sq::skinny2_workspace_bytes(M > 32 ? 32 : M, N, K);
    const size_t b = M > 16 ? sq::gemm_workspace_bytes(M, N, K) : 0;
    return a > b ? a : b;
}

int sq_w4a16_gemm_ws(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int group_size,
                     int layout, int algo, void* workspace, size_t workspace_bytes, void* stream) {
    return gemm_dispatch(x, w, zs, y, M, N, K, group_size, layout, algo, sq::Epilogue{nullptr, nullptr, 0}, workspace,
                         workspace_bytes, stream);
}

// Kernel words worth timing for a shape: every family that can run it, with the tunings its launcher accepts.
// A word the launcher refuses (a K split that does not divide, a missing workspace) is skipped by the caller.
static int autotune_candidates(int M, int K, int g, bool has_ws, int* out, int cap) {
    int n = 0;
    auto add = [&](int kernel, int tune) {
        if (n < cap) out[n++] = kernel | (tune << 8);
    };
    if (M <= 8)
        for (int ks = 1; ks <= 4; ks *= 2)
            for (int nr = 2; nr <= 8; nr *= 2)
                if (nr * ks <= 16) add(SQ_ALGO_GEMV_FIXUP, nr | (ks << 4));
    if (M <= 16 && (g == 128 || g == 64) && K % 128 == 0) {
        const int rows[3] = {1, 3, 4};
        for (int r = 0; r < 3; r++)
            for (int ks = 1; ks <= 8; ks *= 2)
                if (ks == 1 ? K <= 4096 : (has_ws && K / ks >= 1024 && K / ks <= 4096)) add(SQ_ALGO_STREAM, rows[r] | (ks << 4));
    }
    if (M > 16 && M <= 32 && g == 128) add(SQ_ALGO_STREAM, 0);
    if (M > 2 && M <= 32 && has_ws)
        for (int ks = 1; ks <= 8; ks *= 2) add(SQ_ALGO_SKINNY_WS, ks);
    if (M > 2 && M <= 64) add(SQ_ALGO_SKINNY, 0);
    if (M > 16) {
        for (int lds = 0; lds <= (K % 256 == 0 ? 1 : 0); lds++)
            for (int mi = 1; mi <= 4; mi *= 2) {
                if (M <= 64 && mi == 4) continue;
                for (int ks = 1; ks <= (has_ws ? 8 : 1); ks *= 2) add(SQ_ALGO_GEMM, mi | (lds ? 0x80 : 0) | (ks << 8));
            }
        if (M > 64)
            for (int v = 8; v <= 10; v++) add(SQ_ALGO_GEMM, v);
    }
    return n;
}

int sq_w4a16_autotune(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int group_size,
                      int layout, void* workspace, size_t workspace_bytes, int copies, size_t w_stride, size_t zs_stride,
                      int reps, void* stream, int* best_algo, float* best_us, float* auto_us) {
    if (M <= 0) return SQ_ERR_BAD_SHAPE;
    if (copies < 1 || copies > 4096 || reps < 1 || reps > 100000) return SQ_ERR_BAD_SHAPE;
    if (copies > 1 && (w_stride % 16 != 0 || zs_stride % 16 != 0 || w_stride < (size_t)N * K / 2)) return SQ_ERR_MISALIGNED;
    const sq::Epilogue none{nullptr, nullptr, 0};
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool has_ws = full_workspace(workspace, workspace_bytes, M, N, K);
    if (!has_ws) {
        workspace = nullptr;
        workspace_bytes = 0;
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        if (e0) (void)hipEventDestroy(e0);
        return SQ_ERR_LAUNCH;
    }
    // One candidate: a launch that has to succeed, a short warm-up, then `reps` launches between two events,
    // walking through the `copies` weights so that a pool larger than the last-level cache is read from HBM.
    auto run = [&](int word, int i) {
        const size_t c = (size_t)(i % copies);
        return gemm_dispatch(x, static_cast<const uint8_t*>(w) + c * w_stride, static_cast<const uint8_t*>(zs) + c * zs_stride,
                             y, M, N, K, group_size, layout, word, none, workspace, workspace_bytes, stream);
    };
    int status = SQ_OK;
    auto time_word = [&](int word, float* us) {
        int rc = run(word, 0);
        if (rc != SQ_OK) return rc;
        // as many untimed launches as timed ones: clocks and caches are in the candidate's own steady state
        for (int i = 1; i < reps; i++) (void)run(word, i);
        if (hipEventRecord(e0, st) != hipSuccess) return (int)SQ_ERR_LAUNCH;
        for (int i = 0; i < reps; i++) rc |= run(word, i + reps);
        if (hipEventRecord(e1, st) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) return (int)SQ_ERR_LAUNCH;
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) return (int)SQ_ERR_LAUNCH;
        *us = ms * 1000.f / (float)reps;
        return rc;
    };
    // the built-in choice first (with any earlier measurement of this shape out of the way)
    float t_auto = 0.f;
    {
        std::lock_guard<std::mutex> lock(g_tuned_mutex);
        const int n = g_tuned_count.load(std::memory_order_relaxed);
        for (int i = 0; i < n; i++) {
            TunedEntry& e = g_tuned[i];
            if (e.M == M && e.N == N && e.K == K && e.g == group_size && e.has_ws == (int)has_ws) e.M = -1;
        }
    }
    for (int i = 0; i < 2 * reps; i++) (void)run(SQ_ALGO_AUTO, i);  // out of the idle state before anything is timed
    status = time_word(SQ_ALGO_AUTO, &t_auto);
    int best = 0;
    float t_best = t_auto;
    if (status == SQ_OK) {
        int words[96];
        const int n = autotune_candidates(M, K, group_size, has_ws, words, 96);
        for (int i = 0; i < n; i++) {
            float t = 0.f;
            const int rc = time_word(words[i], &t);
            if (rc == SQ_ERR_LAUNCH) {
                status = rc;
                break;
            }
            if (rc == SQ_OK && t < t_best) {
                t_best = t;
                best = words[i];
            }
        }
    }
    if (status == SQ_OK && best != 0) {
        // A candidate has to beat the built-in choice twice, the second time against a fresh timing of both (the
        // clocks of this part move with the load, and an early window can read a few percent off).
        float t_auto2 = 0.f, t_best2 = 0.f;
        if (time_word(SQ_ALGO_AUTO, &t_auto2) == SQ_OK && time_word(best, &t_best2) == SQ_OK) {
            if (t_auto2 < t_auto) t_auto = t_auto2;
            if (t_best2 > t_best) t_best = t_best2;
            if (t_best >= 0.99f * t_auto) {
                best = 0;
                t_best = t_auto;
            }
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (status != SQ_OK) return status;
    // leave the caller's output as the chosen kernel writes it
    status = run(best, 0);
    if (status != SQ_OK) return status;
    if (best != 0) {
        std::lock_guard<std::mutex> lock(g_tuned_mutex);
        const int n = g_tuned_count.load(std::memory_order_relaxed);
        if (n < TUNED_MAX) {
            g_tuned[n] = TunedEntry{M, N, K, group_size, (int)has_ws, best, t_best};
            g_tuned_count.store(n + 1, std::memory_order_release);
        }
    }
    if (best_algo) *best_algo = best;
    if (best_us) *best_us = t_best;
    if (auto_us) *auto_us = t_auto;
    return SQ_OK;
}

int sq_w4a16_autotune_clear(void) {
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    const int n = g_tuned_count.load(std::memory_order_relaxed);
    int live = 0;
    for (int i = 0; i < n; i++) {  // readers may be scanning: entries are voided, never moved
        if (g_tuned[i].M >= 0) live++;
        g_tuned[i].M = -1;
    }
    return live;
}

int sq_w4a16_gemm_static_ws(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int group_size,
                            int layout, int algo, void* stream) {
    // Validate before touching the device, so that argument errors launch nothing.
    if (M < 0) return SQ_ERR_BAD_SHAPE;
    const int rc = check_weight(N, K, group_size, layout);
    if (rc != SQ_OK) return rc;
    if (layout != SQ_LAYOUT_L1) return SQ_ERR_BAD_LAYOUT;
    // What the kernels of this token count would take from a workspace: nothing up to 2 tokens (the GEMV has
    // no workspace form), the split-K decode kernels' counters and partial tiles up to 32, the tiled GEMM's K
    // split beyond and where the automatic choice takes it at 17..32.  A shape that wants more than the static
    // buffer is refused rather than served by a slower workspace-free kernel behind the caller's back.
    size_t need = M <= 2 ? 0 : (M <= 32 ? sq::skinny2_workspace_bytes(M, N, K) : sq::gemm_workspace_bytes(M, N, K));
    if (M > 16 && M <= 32 && builtin_choice(M, N, K, group_size, true, true) == SQ_ALGO_GEMM) {
        const size_t b = sq::gemm_workspace_bytes(M, N, K);
        if (b > need) need = b;
    }
    if (need > (size_t)SQ_STATIC_WS_BYTES) return SQ_ERR_STATIC_WS;
    if (M == 0) return SQ_OK;
    if (!x || !w || !zs || !y) return SQ_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(w) || !aligned16(zs) || !aligned16(y)) return SQ_ERR_MISALIGNED;
    void* ws = static_workspace();
    if (!ws) return SQ_ERR_LAUNCH;
    return gemm_dispatch(x, w, zs, y, M, N, K, group_size, layout, algo, sq::Epilogue{nullptr, nullptr, 0}, ws,
                         (size_t)SQ_STATIC_WS_BYTES, stream);
}

int sq_workspace_reset(void* workspace, size_t bytes, void* stream) {
    if (!workspace) return SQ_ERR_NULL_POINTER;
    if (!aligned16(workspace) || bytes % 4 != 0) return SQ_ERR_MISALIGNED;
    if (bytes == 0) return SQ_OK;
    if (bytes > ((size_t)1 << 30)) return SQ_ERR_BAD_SHAPE;
    const int words = (int)(bytes / 4);
    hipLaunchKernelGGL(zero_words_kernel, dim3((words + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<unsigned*>(workspace), words);
    return launch_code(hipGetLastError());
}

int sq_workspace_check(const void* workspace, size_t bytes, void* stream) {
    if (!workspace) return SQ_ERR_NULL_POINTER;
    if (bytes % 4 != 0) return SQ_ERR_MISALIGNED;
    if (bytes > 65536) bytes = 65536;
    static thread_local unsigned host[65536 / 4];
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (hipMemcpyAsync(host, workspace, bytes, hipMemcpyDeviceToHost, st) != hipSuccess) return SQ_ERR_LAUNCH;
    if (hipStreamSynchronize(st) != hipSuccess) return SQ_ERR_LAUNCH;
    for (size_t i = 0; i < bytes / 4; i++)
        if (host[i] != 0u) return SQ_ERR_WORKSPACE;
    return SQ_OK;
}

static void to_problems(const sq_linear_desc* linears, int count, sq::SeqProblem* probs) {
    for (int l = 0; l < count; l++) {
        const sq_linear_desc& d = linears[l];
        probs[l] = sq::SeqProblem{d.x, d.w, d.zs, d.bias, d.residual, d.y, d.N, d.K, d.group_size, d.act, d.depends};
    }
}

// A sequence's workspace: first what the split-K kernels of the launch-per-linear path want (64 KiB of counters
// and the partial tiles; nothing beyond the counters up to 2 tokens), then, 256-byte aligned, the region of the
// one-launch kernel (control block and exchange words), which no other kernel writes.
static size_t sequence_splitk_bytes(const sq_linear_desc* linears, int count, int M) {
    const size_t base = 65536;
    if (!linears || count <= 0 || count > SQ_SEQUENCE_MAX || M <= 2) return base;
    // more than 2 tokens: what sq_w4a16_gemm_ws wants for the largest run of linears that may share a launch
    // (their rows concatenated, each rounded up to a 64-row block) and for every single linear
    long rows = 0;
    int kmax = 0;
    for (int l = 0; l < count; l++) {
        if (linears[l].N <= 0 || linears[l].K <= 0) return base;
        rows += ((long)linears[l].N + 63) / 64 * 64;
        if (linears[l].K > kmax) kmax = linears[l].K;
    }
    if (rows > (1L << 30)) return base;
    const size_t a = (sq_w4a16_workspace_bytes(M, (int)rows, kmax) + 255) & ~(size_t)255;
    return a > base ? a : base;
}

size_t sq_w4a16_gemv_sequence_workspace_bytes(const sq_linear_desc* linears, int count, int M) {
    sq::SeqProblem probs[SQ_SEQUENCE_MAX];
    const bool listed = linears && count > 0 && count <= SQ_SEQUENCE_MAX;
    if (listed) to_problems(linears, count, probs);
    return sequence_splitk_bytes(linears, count, M) + sq::gemv_seq_workspace_bytes(listed ? probs : nullptr, count, M);
}

int sq_w4a16_gemv_sequence_status(const sq_linear_desc* linears, int count, int M, void* workspace,
                                  size_t workspace_bytes, int clear, void* stream) {
    if (!linears || !workspace) return SQ_ERR_NULL_POINTER;
    if (count <= 0 || count > SQ_SEQUENCE_MAX) return SQ_ERR_BAD_SHAPE;
    const size_t off = sequence_splitk_bytes(linears, count, M);
    if (!aligned16(workspace) || workspace_bytes < off + 256) return SQ_ERR_WORKSPACE;
    unsigned* ctrl = reinterpret_cast<unsigned*>(static_cast<uint8_t*>(workspace) + off);
    unsigned host[4] = {0, 0, 0, 0};
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (hipMemcpyAsync(host, ctrl, sizeof(host), hipMemcpyDeviceToHost, st) != hipSuccess) return SQ_ERR_LAUNCH;
    if (hipStreamSynchronize(st) != hipSuccess) return SQ_ERR_LAUNCH;
    if (clear && host[1] != 0u) {
        hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, st, ctrl + 1, 1);
        if (hipGetLastError() != hipSuccess) return SQ_ERR_LAUNCH;
    }
    if (host[2] != 0u) return SQ_ERR_WORKSPACE;  // an exit counter that is not back at zero: a launch did not finish
    return host[1] != 0u ? SQ_ERR_SEQ_TIMEOUT : SQ_OK;
}

// Tuning of the persistent sequence kernel (sq_w4a16_gemv_sequence_tune): polls allowed for another workgroup's
// output, and loads a streaming wave keeps in flight (0: the kernel's default).
static unsigned g_seq_spin_limit = 1u << 16;
static int g_seq_lim = 0;

int sq_w4a16_gemv_sequence_tune(unsigned spin_limit, int loads_in_flight) {
    if (loads_in_flight < 0 || loads_in_flight > 16) return SQ_ERR_BAD_SHAPE;
    g_seq_spin_limit = spin_limit;
    g_seq_lim = loads_in_flight;
    return SQ_OK;
}

int sq_w4a16_gemv_sequence(const sq_linear_desc* linears, int count, int M, int layout, int mode, void* workspace,
                           size_t workspace_bytes, void* stream) {
    if (count < 0 || count > SQ_SEQUENCE_MAX) return SQ_ERR_BAD_SHAPE;
    if (mode != SQ_SEQ_AUTO && mode != SQ_SEQ_ONE_LAUNCH) return SQ_ERR_BAD_ALGO;
    if (count == 0) return SQ_OK;
    if (!linears) return SQ_ERR_NULL_POINTER;
    if (M < 0) return SQ_ERR_BAD_SHAPE;
    if (layout != SQ_LAYOUT_L1) return SQ_ERR_BAD_LAYOUT;
    sq::SeqProblem probs[SQ_SEQUENCE_MAX];
    for (int l = 0; l < count; l++) {
        const sq_linear_desc& d = linears[l];
        const int rc = check_weight(d.N, d.K, d.group_size, layout);
        if (rc != SQ_OK) return rc;
        if (d.act != SQ_ACT_NONE && d.act != SQ_ACT_RELU) return SQ_ERR_BAD_ALGO;
        if (M > 0) {
            if (!d.x || !d.w || !d.zs || !d.y) return SQ_ERR_NULL_POINTER;
            if (!aligned16(d.x) || !aligned16(d.w) || !aligned16(d.zs) || !aligned16(d.y)) return SQ_ERR_MISALIGNED;
            if ((d.bias && (reinterpret_cast<uintptr_t>(d.bias) & 1u)) ||
                (d.residual && (reinterpret_cast<uintptr_t>(d.residual) & 1u)))
                return SQ_ERR_MISALIGNED;
        }
        probs[l] = sq::SeqProblem{d.x, d.w, d.zs, d.bias, d.residual, d.y, d.N, d.K, d.group_size, d.act, d.depends};
    }
    if (M == 0) return SQ_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (workspace && !aligned16(workspace)) workspace = nullptr;
    if (mode == SQ_SEQ_ONE_LAUNCH && workspace && M <= 4) {
        // everything in one persistent launch; outputs that later linears read travel as tagged words
        const size_t off = sequence_splitk_bytes(linears, count, M);
        const int rc = workspace_bytes > off ? sq::launch_gemv_seq(probs, count, M, static_cast<uint8_t*>(workspace) + off,
                                                                   workspace_bytes - off, g_seq_spin_limit, g_seq_lim, st)
                                             : 1;
        if (rc == 0) return SQ_OK;
        if (rc == 2) return SQ_ERR_LAUNCH;
    }
    // A linear that depends on an earlier one starts a new launch: the kernel boundary is the cheapest way to
    // honour a dependency on this part (about 2 us, against 5..9 us for a grid barrier inside a persistent
    // kernel).  Consecutive linears that do not depend on each other and share K and the group size (q, k and
    // v of a decoder layer) go out as ONE launch of the single-linear GEMV whose grid is the concatenation of
    // their row blocks.  Everything else (more than 4 tokens, K beyond 8192, a lone linear) is one launch per
    // linear through the automatic dispatch.
    int l0 = 0;
    while (l0 < count) {
        int l1 = l0 + 1;
        while (l1 < count && l1 - l0 < sq::GEMV_GROUP_MAX && !probs[l1].depends && probs[l1].K == probs[l0].K &&
               probs[l1].group_size == probs[l0].group_size)
            l1++;
        bool done = false;
        if (l1 - l0 > 1 && M <= 4 && probs[l0].K <= 8192) {
            const hipError_t e = sq::launch_gemv2_group(probs + l0, l1 - l0, M, st);
            if (e == hipSuccess)
                done = true;
            else if (e != hipErrorInvalidValue)
                return SQ_ERR_LAUNCH;
        } else if (l1 - l0 > 1 && M > 4 && M <= 16 && probs[l0].group_size == 128 && probs[l0].K % 128 == 0 &&
                   (probs[l0].K <= 4096 || workspace)) {
            // the streaming decode kernel on the concatenated row blocks (a K beyond 4096 needs the workspace)
            const hipError_t e = sq::launch_skinny3_group(probs + l0, l1 - l0, M, workspace, workspace_bytes, st);
            if (e == hipSuccess)
                done = true;
            else if (e != hipErrorInvalidValue)
                return SQ_ERR_LAUNCH;
        }
        if (!done && l1 - l0 > 1 && M > 16 && M <= 32 && probs[l0].group_size == 128 && probs[l0].K % 128 == 0 &&
            (probs[l0].K <= 4096 || workspace)) {
            const hipError_t e = sq::launch_skinny3_wide_group(probs + l0, l1 - l0, M, workspace, workspace_bytes, st);
            if (e == hipSuccess)
                done = true;
            else if (e != hipErrorInvalidValue)
                return SQ_ERR_LAUNCH;
        }
        if (!done && l1 - l0 > 1 && M > 4 && M <= 32 && workspace && aligned16(workspace)) {
            // the split-K decode kernel on the concatenated row blocks, where it is what one linear of the
            // group's total size would get (large weight, more than 16 tokens, or long K)
            long elems = 0;
            for (int l = l0; l < l1; l++) elems += (long)probs[l].N * probs[l].K;
            if (elems >= (1L << 25) || M > 16 || probs[l0].K > 8192) {
                const hipError_t e = sq::launch_skinny2_group(probs + l0, l1 - l0, M, workspace, workspace_bytes, st);
                if (e == hipSuccess)
                    done = true;
                else if (e != hipErrorInvalidValue)
                    return SQ_ERR_LAUNCH;
            }
        }
        if (!done) {
            for (int l = l0; l < l1; l++) {
                const sq::SeqProblem& q = probs[l];
                const sq::Epilogue epi{static_cast<const sq::half_t*>(q.bias), static_cast<const sq::half_t*>(q.residual),
                                       q.act};
                const int rc = gemm_dispatch(q.x, q.w, q.zs, q.y, M, q.N, q.K, q.group_size, layout, SQ_ALGO_AUTO, epi,
                                             M > 2 ? workspace : nullptr, M > 2 ? workspace_bytes : 0, stream);
                if (rc != SQ_OK) return rc;
            }
        }
        l0 = l1;
    }
    return SQ_OK;
}

int sq_w4a16_gemm_fused(const void* x, const void* w, const void* zs, const void* bias, const void* residual, void* y,
                        int M, int N, int K, int group_size, int layout, int act, int algo, void* workspace,
                        size_t workspace_bytes, void* stream) {
    if (act != SQ_ACT_NONE && act != SQ_ACT_RELU && act != SQ_ACT_SILU) return SQ_ERR_BAD_ALGO;
    if (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)) return SQ_ERR_MISALIGNED;
    if (residual && (reinterpret_cast<uintptr_t>(residual) & 1u)) return SQ_ERR_MISALIGNED;
    const sq::Epilogue epi{static_cast<const sq::half_t*>(bias), static_cast<const sq::half_t*>(residual), act};
    return gemm_dispatch(x, w, zs, y, M, N, K, group_size, layout, algo, epi, workspace, workspace_bytes, stream);
}

int sq_w4a16_gemm_silu_dot(const void* x, const void* w_gate, const void* zs_gate, const void* w_up, const void* zs_up,
                           void* y, void* up_scratch, int M, int N, int K, int group_size, int layout, void* workspace,
                           size_t workspace_bytes, void* stream) {
    if (M > 0 && (!up_scratch || !w_up || !zs_up)) return SQ_ERR_NULL_POINTER;
    if (M > 0 && !aligned16(up_scratch)) return SQ_ERR_MISALIGNED;
    if (M > 0 && up_scratch == y) return SQ_ERR_BAD_SHAPE;
    // the up projection first, rounded to fp16 once; the gate projection multiplies it into its store
    const int rc = gemm_dispatch(x, w_up, zs_up, up_scratch, M, N, K, group_size, layout, SQ_ALGO_AUTO,
                                 sq::Epilogue{nullptr, nullptr, SQ_ACT_NONE}, workspace, workspace_bytes, stream);
    if (rc != SQ_OK || M == 0) return rc;
    sq::Epilogue epi{nullptr, nullptr, SQ_ACT_SILU};
    epi.mul = static_cast<const sq::half_t*>(up_scratch);
    return gemm_dispatch(x, w_gate, zs_gate, y, M, N, K, group_size, layout, SQ_ALGO_AUTO, epi, workspace,
                         workspace_bytes, stream);
}

int sq_w4a16_gemm(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int group_size,
                  int layout, void* stream) {
    return sq_w4a16_gemm_ex(x, w, zs, y, M, N, K, group_size, layout, SQ_ALGO_AUTO, stream);
}

int sq_w4a16_dequant(const void* w, const void* zs, void* out, int N, int K, int group_size, int layout,
                     void* stream) {
    const int rc = check_weight(N, K, group_size, layout);
    if (rc != SQ_OK) return rc;
    if (!w || !zs || !out) return SQ_ERR_NULL_POINTER;
    if (!aligned16(w) || !aligned16(zs) || !aligned16(out)) return SQ_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (layout == SQ_LAYOUT_L1) return launch_code(sq::launch_dequant_l1(w, zs, out, N, K, group_size, st));
    return launch_code(sq::launch_dequant_l2(w, zs, out, N, K, group_size, st));
}

int sq_transpose_merge_zeros_scales(const void* zeros, const void* scales, void* zs, int in_features,
                                    int out_features, int group_size, void* stream) {
    if (in_features <= 0 || out_features <= 0) return SQ_ERR_BAD_SHAPE;
    if (group_size <= 0 || in_features % group_size != 0) return SQ_ERR_BAD_GROUP;
    if (!zeros || !scales || !zs) return SQ_ERR_NULL_POINTER;
    return launch_code(sq::launch_transpose_merge_zeros_scales(zeros, scales, zs, in_features, out_features,
                                                               group_size, static_cast<hipStream_t>(stream)));
}

int sq_convert_ours_to_awq(const void* src, void* dst, int in_features, int out_features, void* stream) {
    if (in_features <= 0 || out_features <= 0 || in_features % 2 != 0 || out_features % 8 != 0)
        return SQ_ERR_BAD_SHAPE;
    if (!src || !dst) return SQ_ERR_NULL_POINTER;
    return launch_code(
        sq::launch_ours_to_awq(src, dst, in_features, out_features, static_cast<hipStream_t>(stream)));
}

int sq_convert_awq_to_lmdeploy(const void* src, void* dst, int in_features, int out_features, void* stream) {
    if (in_features <= 0 || out_features <= 0 || in_features % 32 != 0 || out_features % 32 != 0)
        return SQ_ERR_BAD_SHAPE;
    if (!src || !dst) return SQ_ERR_NULL_POINTER;
    if (src == dst) return SQ_ERR_BAD_SHAPE;
    return launch_code(
        sq::launch_awq_to_lmdeploy(src, dst, in_features, out_features, static_cast<hipStream_t>(stream)));
}

int sq_repack_l2_to_l1(const void* w_l2, const void* zs_l2, void* w_l1, void* zs_l1, int N, int K, int group_size,
                       void* stream) {
    const int rc = check_weight(N, K, group_size, SQ_LAYOUT_L2);
    if (rc != SQ_OK) return rc;
    if (!w_l2 || !zs_l2 || !w_l1 || !zs_l1) return SQ_ERR_NULL_POINTER;
    return launch_code(
        sq::launch_l2_to_l1(w_l2, zs_l2, w_l1, zs_l1, N, K, group_size, static_cast<hipStream_t>(stream)));
}

int sq_convert_2bit_to_4bit(const void* src, void* dst, int N, int K, void* stream) {
    if (N <= 0 || K <= 0 || K % 4 != 0) return SQ_ERR_BAD_SHAPE;
    if (!src || !dst) return SQ_ERR_NULL_POINTER;
    return launch_code(sq::launch_2bit_to_4bit(src, dst, N, K, static_cast<hipStream_t>(stream)));
}

int sq_l2_convert_4bit_to_2bit(const void* src, void* dst, int K, int N, void* stream) {
    if (N <= 0 || K <= 0 || N % 16 != 0) return SQ_ERR_BAD_SHAPE;
    if (!src || !dst) return SQ_ERR_NULL_POINTER;
    return launch_code(sq::launch_l2_4bit_to_2bit(src, dst, K, N, static_cast<hipStream_t>(stream)));
}

int sq_l2_convert_2bit_to_4bit(const void* src, void* dst, int K, int N, void* stream) {
    if (N <= 0 || K <= 0 || N % 16 != 0) return SQ_ERR_BAD_SHAPE;
    if (!src || !dst) return SQ_ERR_NULL_POINTER;
    return launch_code(sq::launch_l2_2bit_to_4bit(src, dst, K, N, static_cast<hipStream_t>(stream)));
}

int sq_lut_attention_fwd(const void* q, const void* k, const void* v, void* out, const void* lut, int lut_elem_bytes,
                         int Z, int H, int S, int D, int nnz, float sm_scale, int causal, void* stream) {
    if (Z <= 0 || H <= 0 || S <= 0 || nnz <= 0 || (D != 64 && D != 128)) return SQ_ERR_BAD_SHAPE;
    if ((long)Z * H > 65535) return SQ_ERR_BAD_SHAPE;
    if (lut_elem_bytes != 4 && lut_elem_bytes != 8) return SQ_ERR_BAD_LAYOUT;
    if (!q || !k || !v || !out || !lut) return SQ_ERR_NULL_POINTER;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return SQ_ERR_MISALIGNED;
    return launch_code(sq::launch_lut_attention(q, k, v, out, lut, lut_elem_bytes, Z, H, S, D, nnz, sm_scale, causal,
                                                static_cast<hipStream_t>(stream)));
}

int sq_decode_attention(const void* q, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                        const void* mask, void* out, int B, int H, int D, int Lmax, long q_bstride, long q_hstride,
                        long new_bstride, long new_hstride, long cache_bstride, long cache_hstride, long mask_bstride,
                        int cache_len, const long long* cache_len_dev, float sm_scale, void* workspace,
                        size_t workspace_bytes, void* stream) {
    if (B <= 0 || H <= 0 || Lmax <= 0 || (D != 64 && D != 128)) return SQ_ERR_BAD_SHAPE;
    if ((long)B * H > (1L << 24)) return SQ_ERR_BAD_SHAPE;
    if (!q || !k_cache || !v_cache || !out) return SQ_ERR_NULL_POINTER;
    if ((k_new == nullptr) != (v_new == nullptr)) return SQ_ERR_NULL_POINTER;
    const bool append = k_new != nullptr;
    if (!cache_len_dev) {  // a length on the device is clamped to the cache by the kernel
        if (cache_len < 0 || cache_len + (append ? 1 : 0) > Lmax || cache_len + (append ? 1 : 0) < 1)
            return SQ_ERR_BAD_SHAPE;
    }
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || (append && (!aligned16(k_new) || !aligned16(v_new))))
        return SQ_ERR_MISALIGNED;
    if ((q_bstride | q_hstride | cache_bstride | cache_hstride) % 8 != 0) return SQ_ERR_MISALIGNED;
    if (append && (new_bstride | new_hstride) % 8 != 0) return SQ_ERR_MISALIGNED;
    if (q_bstride < 0 || q_hstride < 0 || cache_bstride < 0 || cache_hstride < (long)Lmax * D || mask_bstride < 0 ||
        (append && (new_bstride < 0 || new_hstride < 0)))
        return SQ_ERR_BAD_SHAPE;
    return launch_code(sq::launch_decode_attention(q, k_new, v_new, k_cache, v_cache, mask, out, B, H, D, Lmax,
                                                   q_bstride, q_hstride, new_bstride, new_hstride, cache_bstride,
                                                   cache_hstride, mask_bstride, cache_len, cache_len_dev, sm_scale,
                                                   aligned16(workspace) ? workspace : nullptr, workspace_bytes,
                                                   static_cast<hipStream_t>(stream)));
}

size_t sq_decode_attention_workspace_bytes(int B, int H, int D) {
    if (B <= 0 || H <= 0 || (D != 64 && D != 128)) return 0;
    return sq::decode_attention_workspace_bytes(B, H, D);
}

int sq_layernorm(const void* x, const void* gamma, const void* beta, void* y, int rows, int cols, float eps,
                 void* stream) {
    if (rows < 0 || cols <= 0 || cols % 8 != 0 || cols > 16384) return SQ_ERR_BAD_SHAPE;
    if (rows == 0) return SQ_OK;
    if (!x || !y) return SQ_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(y) || (gamma && !aligned16(gamma)) || (beta && !aligned16(beta)))
        return SQ_ERR_MISALIGNED;
    return launch_code(sq::launch_layernorm(x, gamma, beta, y, rows, cols, eps, static_cast<hipStream_t>(stream)));
}

int sq_w4a16_ln_fusable(int M, int N, int K, int group_size, int layout) {
    return layout == SQ_LAYOUT_L1 && M >= 1 && M <= 8 && N > 0 && group_size == 128 && K % 128 == 0 && K > 2048 &&
                   K <= 4096
               ? 1
               : 0;
}

int sq_w4a16_gemm_ln_fused(const void* x, const void* ln_gamma, const void* ln_beta, float ln_eps, void* x_norm,
                           const void* w, const void* zs, const void* bias, const void* residual, void* y, int M, int N,
                           int K, int group_size, int layout, int act, void* workspace, size_t workspace_bytes,
                           void* stream) {
    if (act != SQ_ACT_NONE && act != SQ_ACT_RELU && act != SQ_ACT_SILU) return SQ_ERR_BAD_ALGO;
    if (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)) return SQ_ERR_MISALIGNED;
    if (residual && (reinterpret_cast<uintptr_t>(residual) & 1u)) return SQ_ERR_MISALIGNED;
    if ((ln_gamma && !aligned16(ln_gamma)) || (ln_beta && !aligned16(ln_beta))) return SQ_ERR_MISALIGNED;
    if (M < 0) return SQ_ERR_BAD_SHAPE;
    const int rc = check_weight(N, K, group_size, layout);
    if (rc != SQ_OK) return rc;
    if (layout != SQ_LAYOUT_L1) return SQ_ERR_BAD_LAYOUT;
    if (M == 0) return SQ_OK;
    const sq::Epilogue epi{static_cast<const sq::half_t*>(bias), static_cast<const sq::half_t*>(residual), act};
    if (sq_w4a16_ln_fusable(M, N, K, group_size, layout)) {
        if (!x || !w || !zs || !y) return SQ_ERR_NULL_POINTER;
        if (!aligned16(x) || !aligned16(w) || !aligned16(zs) || !aligned16(y)) return SQ_ERR_MISALIGNED;
        const sq::LnPre ln{static_cast<const sq::half_t*>(ln_gamma), static_cast<const sq::half_t*>(ln_beta), ln_eps};
        const hipError_t e = sq::launch_skinny3_tuned(x, w, zs, y, nullptr, M, N, K, group_size, 0, epi, &ln,
                                                      static_cast<hipStream_t>(stream));
        if (e != hipErrorInvalidValue) return launch_code(e);
    }
    // Not fusable: the LayerNorm kernel into the caller's scratch rows, then the linear on those.
    if (!x_norm) return SQ_ERR_NULL_POINTER;
    if (K > 16384) return SQ_ERR_BAD_SHAPE;
    const int rl = sq_layernorm(x, ln_gamma, ln_beta, x_norm, M, K, ln_eps, stream);
    if (rl != SQ_OK) return rl;
    return gemm_dispatch(x_norm, w, zs, y, M, N, K, group_size, layout, SQ_ALGO_AUTO, epi, workspace, workspace_bytes,
                         stream);
}

int sq_embed_rows(const void* embed, const void* pos_table, const void* tok, const void* pos, long long pos_offset,
                  void* out, int rows, int hidden, long long vocab, long long positions, void* stream) {
    if (rows < 0 || hidden <= 0 || hidden % 8 != 0 || vocab <= 0 || positions <= 0) return SQ_ERR_BAD_SHAPE;
    if (rows == 0) return SQ_OK;
    if (!embed || !pos_table || !tok || !pos || !out) return SQ_ERR_NULL_POINTER;
    if (!aligned16(embed) || !aligned16(pos_table) || !aligned16(out) || (reinterpret_cast<uintptr_t>(tok) & 7u) ||
        (reinterpret_cast<uintptr_t>(pos) & 7u))
        return SQ_ERR_MISALIGNED;
    return launch_code(sq::launch_embed_rows(embed, pos_table, tok, pos, pos_offset, out, rows, hidden, vocab, positions,
                                             static_cast<hipStream_t>(stream)));
}

int sq_f16_gemv_parts(int N) { return N > 0 ? sq::f16_gemv_parts(N) : 0; }

int sq_f16_gemv(const void* x, const void* w, void* y, void* part_val, void* part_idx, int M, int N, int K, void* stream) {
    if (M < 0 || M > 8 || N <= 0 || K < 512 || K % 512 != 0 || K > 8192) return SQ_ERR_BAD_SHAPE;
    if (M == 0) return SQ_OK;
    if (!x || !w || !y || ((part_val == nullptr) != (part_idx == nullptr))) return SQ_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(w) || (reinterpret_cast<uintptr_t>(y) & 1u) ||
        (reinterpret_cast<uintptr_t>(part_val) & 3u) || (reinterpret_cast<uintptr_t>(part_idx) & 3u))
        return SQ_ERR_MISALIGNED;
    return launch_code(sq::launch_f16_gemv(x, w, y, static_cast<float*>(part_val), static_cast<int*>(part_idx), M, N, K,
                                           static_cast<hipStream_t>(stream)));
}

int sq_greedy_feedback(const void* part_val, const void* part_idx, int parts, int M, void* tok, void* pos, void* history,
                       void* step, long long history_rows, void* stream) {
    if (M < 0 || M > 8 || parts <= 0 || history_rows < 0) return SQ_ERR_BAD_SHAPE;
    if (M == 0) return SQ_OK;
    if (!part_val || !part_idx || !tok) return SQ_ERR_NULL_POINTER;
    if ((reinterpret_cast<uintptr_t>(tok) & 7u) || (reinterpret_cast<uintptr_t>(pos) & 7u) ||
        (reinterpret_cast<uintptr_t>(history) & 7u) || (reinterpret_cast<uintptr_t>(step) & 7u))
        return SQ_ERR_MISALIGNED;
    return launch_code(sq::launch_greedy_feedback(static_cast<const float*>(part_val), static_cast<const int*>(part_idx),
                                                  parts, M, tok, pos, history, step, history_rows,
                                                  static_cast<hipStream_t>(stream)));
}

}  // extern "C"
