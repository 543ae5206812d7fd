// `quant`: the PyTorch-ROCm extension module the reference's Python code imports
// (`from quant import gemm_awq_ut, dequant, transpose_merge_zeros_scales, ...`).
// Host C++ only: it validates tensors the way the reference does, takes torch's
// current HIP stream and forwards raw pointers to the C ABI of libsq_w4a16.so.
//
// Reference interfaces mirrored here:
//   gemm_awq_ut / Gemm_awq_pure   quantization/nvidia/kernel/gemm_quant.cu:42-123,
//                                 quantization/muxi/backend/gemm_quant.cu:12-109
//   dequant                       quantization/tianshu/backend/gemm_quant.cu:153-164
//   transpose_merge_zeros_scales, convert_ours_to_awq, convert_awq_to_lmdeploy
//                                 quantization/nvidia/kernel/gemm_s4_f16/format.cu:135-239
//   module definition             quantization/{nvidia/kernel,muxi/backend,tianshu/backend}/pybind.cpp
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <map>
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>

#include "sq_w4a16.h"

namespace {

#define SQ_CHECK_DEVICE(x) TORCH_CHECK((x).is_cuda(), "Tensor " #x " must be on CUDA")
#define SQ_CHECK_CONTIGUOUS(x) TORCH_CHECK((x).is_contiguous(), "Tensor " #x " must be contiguous")
#define SQ_CHECK_DTYPE(x, t) TORCH_CHECK((x).dtype() == (t), "Tensor " #x " must have dtype (" #t ")")
#define SQ_CHECK_DIMS(x, d) TORCH_CHECK((x).dim() == (d), "Tensor " #x " must have dimension number (" #d ")")

void* current_stream(const at::Tensor& t) {
    return static_cast<void*>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

void raise_if_error(int code, const char* what) {
    if (code == SQ_OK) return;
    const std::string msg = std::string(what) + ": " + sq_strerror(code);
    // Shape / group complaints surface as ValueError like the wave64 back-ends'
    // std::invalid_argument; everything else as RuntimeError like TORCH_CHECK.
    if (code == SQ_ERR_BAD_SHAPE) throw std::invalid_argument(msg);
    throw std::runtime_error(msg);
}

int layout_of(const at::Tensor& W) {
    if (W.scalar_type() == at::kByte) return SQ_LAYOUT_L1;
    if (W.scalar_type() == at::kInt) return SQ_LAYOUT_L2;
    TORCH_CHECK(false, "Tensor W must have dtype uint8 ([N, K/2], wave64 layout) or int32 ([K, N/8], "
                       "tensor-core layout)");
    return 0;
}

// Layout-L2 weights are converted to L1 once and kept while the source tensors
// live.  The key is the weight's data pointer; an entry is valid only while the
// storages of both sources (weight and zeros_scales) are alive (weak references),
// unmodified (version counters) and the same zeros_scales tensor is passed again.
// The conversion is enqueued on the stream of the first call; an event recorded
// behind it orders a later call on another stream after it.
struct RepackEntry {
    c10::weak_intrusive_ptr<c10::StorageImpl> src_storage, zs_storage;
    int64_t version, zs_version;
    const void* zs_ptr;
    void* stream;
    hipEvent_t done;
    at::Tensor w_l1, zs_l1;
};
std::mutex g_cache_mutex;
std::unordered_map<const void*, RepackEntry> g_repack_cache;

void drop_entry(RepackEntry& e) {
    if (e.done) (void)hipEventDestroy(e.done);
    e.done = nullptr;
}

void sweep_cache_locked() {
    for (auto it = g_repack_cache.begin(); it != g_repack_cache.end();) {
        if (it->second.src_storage.expired() || it->second.zs_storage.expired()) {
            drop_entry(it->second);
            it = g_repack_cache.erase(it);
        } else {
            ++it;
        }
    }
}

std::pair<at::Tensor, at::Tensor> l1_view_of_l2(const at::Tensor& W, const at::Tensor& ZS, int N, int K, int g) {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    const void* key = W.data_ptr();
    void* stream = current_stream(W);
    auto it = g_repack_cache.find(key);
    if (it != g_repack_cache.end()) {
        RepackEntry& e = it->second;
        if (!e.src_storage.expired() && !e.zs_storage.expired() && e.version == (int64_t)W._version() &&
            e.zs_ptr == ZS.data_ptr() && e.zs_version == (int64_t)ZS._version() && e.w_l1.size(0) == N &&
            e.w_l1.size(1) == K / 2 && e.zs_l1.size(1) == 2 * (K / g)) {
            if (stream != e.stream && e.done) {
                if (hipStreamWaitEvent(static_cast<hipStream_t>(stream), e.done, 0) != hipSuccess)
                    throw std::runtime_error("repack: hipStreamWaitEvent failed");
            }
            return {e.w_l1, e.zs_l1};
        }
        drop_entry(e);
        g_repack_cache.erase(it);
    }
    sweep_cache_locked();
    at::Tensor w1 = torch::empty({N, K / 2}, W.options().dtype(at::kByte));
    at::Tensor zs1 = torch::empty({N, 2 * (K / g)}, ZS.options());
    raise_if_error(sq_repack_l2_to_l1(W.data_ptr(), ZS.data_ptr(), w1.data_ptr(), zs1.data_ptr(), N, K, g, stream),
                   "repack");
    hipEvent_t done = nullptr;
    if (hipEventCreateWithFlags(&done, hipEventDisableTiming) != hipSuccess ||
        hipEventRecord(done, static_cast<hipStream_t>(stream)) != hipSuccess)
        throw std::runtime_error("repack: could not record the completion event");
    RepackEntry e{c10::weak_intrusive_ptr<c10::StorageImpl>(W.storage().getWeakStorageImpl()),
                  c10::weak_intrusive_ptr<c10::StorageImpl>(ZS.storage().getWeakStorageImpl()),
                  (int64_t)W._version(), (int64_t)ZS._version(), ZS.data_ptr(), stream, done, w1, zs1};
    g_repack_cache.emplace(key, std::move(e));
    return {w1, zs1};
}

// Workspace of the split-K kernels (5..1024 tokens): one zero-initialised buffer per
// (device, stream), grown on demand and kept for the life of the process.  Calls on one
// stream are ordered, which is what sharing a workspace requires.  Under HIP graph capture
// the buffer must already exist (run the call once on the capturing stream beforehand).
std::mutex g_ws_mutex;
std::map<std::pair<int, void*>, at::Tensor> g_workspaces;
std::vector<at::Tensor> g_retired;

at::Tensor workspace_for(const at::Tensor& like, void* stream, size_t bytes) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    const auto key = std::make_pair((int)like.device().index(), stream);
    auto it = g_workspaces.find(key);
    if (it != g_workspaces.end() && (size_t)it->second.numel() >= bytes) return it->second;
    const int64_t want = (int64_t)std::max<size_t>(bytes, (size_t)1 << 20);
    at::Tensor ws = torch::zeros({want}, like.options().dtype(at::kByte));
    // A captured HIP graph may still hold the address of the smaller buffer: keep it alive.
    if (it != g_workspaces.end()) g_retired.push_back(it->second);
    g_workspaces[key] = ws;
    return ws;
}

// LayerNorm in front of the linear (weight / bias fp16 [K] or absent).
struct LnArgs {
    c10::optional<at::Tensor> weight, bias;
    double eps;
};

at::Tensor gemm_impl(const at::Tensor& I, const at::Tensor& W, const at::Tensor& ZS, int N, int group_size, int algo,
                     const c10::optional<at::Tensor>& bias = c10::nullopt,
                     const c10::optional<at::Tensor>& residual = c10::nullopt, int act = SQ_ACT_NONE,
                     const LnArgs* ln = nullptr) {
    SQ_CHECK_DEVICE(I);
    SQ_CHECK_DEVICE(W);
    SQ_CHECK_DEVICE(ZS);
    SQ_CHECK_CONTIGUOUS(I);
    SQ_CHECK_CONTIGUOUS(W);
    SQ_CHECK_CONTIGUOUS(ZS);
    SQ_CHECK_DTYPE(I, at::kHalf);
    SQ_CHECK_DTYPE(ZS, at::kHalf);
    SQ_CHECK_DIMS(I, 3);
    SQ_CHECK_DIMS(W, 2);
    SQ_CHECK_DIMS(ZS, 2);
    const int layout = layout_of(W);
    const int64_t M = I.size(0) * I.size(1);
    const int64_t K = I.size(2);
    if (group_size <= 0 || K % group_size != 0) throw std::invalid_argument("embbed dim must be a multiple of group_size!");
    if (layout == SQ_LAYOUT_L1) {
        if (W.size(0) != N) throw std::invalid_argument("output dim mismatch!");
        if (W.size(1) * 2 != K) throw std::invalid_argument("input dim mismatch!");
        if (ZS.size(0) != N || ZS.size(1) != 2 * (K / group_size))
            throw std::invalid_argument("zeros_scales shape mismatch!");
    } else {
        if (W.size(0) != K) throw std::invalid_argument("input dim mismatch!");
        if (W.size(1) * 8 != N) throw std::invalid_argument("output dim mismatch!");
        if (group_size != 128) throw std::runtime_error("unsupported group size");
        if (ZS.size(0) != K / group_size || ZS.size(1) != 2 * (int64_t)N)
            throw std::invalid_argument("zeros_scales shape mismatch!");
    }
    TORCH_CHECK(M < (1LL << 31) && K < (1LL << 31), "problem too large");

    c10::DeviceGuard guard(I.device());
    at::Tensor O = torch::empty({I.size(0), I.size(1), N}, I.options());
    const void* w_ptr = W.data_ptr();
    const void* zs_ptr = ZS.data_ptr();
    std::pair<at::Tensor, at::Tensor> keep;
    if (layout == SQ_LAYOUT_L2) {
        keep = l1_view_of_l2(W, ZS, N, (int)K, group_size);
        w_ptr = keep.first.data_ptr();
        zs_ptr = keep.second.data_ptr();
    }
    const void* bias_ptr = nullptr;
    const void* res_ptr = nullptr;
    if (bias.has_value() && bias->defined()) {
        SQ_CHECK_DEVICE((*bias));
        SQ_CHECK_CONTIGUOUS((*bias));
        SQ_CHECK_DTYPE((*bias), at::kHalf);
        if (bias->numel() != N) throw std::invalid_argument("bias must have N elements!");
        bias_ptr = bias->data_ptr();
    }
    if (residual.has_value() && residual->defined()) {
        SQ_CHECK_DEVICE((*residual));
        SQ_CHECK_CONTIGUOUS((*residual));
        SQ_CHECK_DTYPE((*residual), at::kHalf);
        if (residual->numel() != M * (int64_t)N) throw std::invalid_argument("residual must have M*N elements!");
        res_ptr = residual->data_ptr();
    }
    void* stream = current_stream(I);
    void* ws_ptr = nullptr;
    size_t ws_bytes = 0;
    at::Tensor ws;
    if (M > 2 && M <= 1024 && ((algo & 0xFF) == SQ_ALGO_AUTO || (algo & 0xFF) == SQ_ALGO_SKINNY_WS || (algo & 0xFF) == SQ_ALGO_STREAM)) {
        ws = workspace_for(I, stream, sq_w4a16_workspace_bytes((int)M, N, (int)K));
        ws_ptr = ws.data_ptr();
        ws_bytes = (size_t)ws.numel();
    }
    if (ln) {
        const void* g_ptr = nullptr;
        const void* b_ptr = nullptr;
        for (int which = 0; which < 2; which++) {
            const c10::optional<at::Tensor>& t = which ? ln->bias : ln->weight;
            if (!t.has_value() || !t->defined()) continue;
            SQ_CHECK_DEVICE((*t));
            SQ_CHECK_CONTIGUOUS((*t));
            SQ_CHECK_DTYPE((*t), at::kHalf);
            if (t->numel() != K) throw std::invalid_argument("LayerNorm parameters must have K elements!");
            (which ? b_ptr : g_ptr) = t->data_ptr();
        }
        at::Tensor scratch;  // normalised rows, only where the kernel cannot normalise in place
        if (!sq_w4a16_ln_fusable((int)M, N, (int)K, group_size, SQ_LAYOUT_L1)) scratch = torch::empty_like(I);
        raise_if_error(sq_w4a16_gemm_ln_fused(I.data_ptr(), g_ptr, b_ptr, (float)ln->eps,
                                              scratch.defined() ? scratch.data_ptr() : nullptr, w_ptr, zs_ptr, bias_ptr,
                                              res_ptr, O.data_ptr(), (int)M, N, (int)K, group_size, SQ_LAYOUT_L1, act,
                                              ws_ptr, ws_bytes, stream),
                       "gemm_awq_ln_fused_ut");
        return O;
    }
    raise_if_error(sq_w4a16_gemm_fused(I.data_ptr(), w_ptr, zs_ptr, bias_ptr, res_ptr, O.data_ptr(), (int)M, N, (int)K,
                                       group_size, SQ_LAYOUT_L1, act, algo, ws_ptr, ws_bytes, stream),
                   "gemm_awq_ut");
    return O;
}

// I [bs, seq, K] fp16; W / W_zeros_scales in layout L1 or L2; returns [bs, seq, N].
// As in the reference the M and K arguments are not used: M is bs*seq and K is
// I.size(2).
at::Tensor gemm_awq_ut(at::Tensor I, at::Tensor W, at::Tensor W_zeros_scales, const int M, const int N,
                       const int K, const int group_size) {
    (void)M;
    (void)K;
    return gemm_impl(I, W, W_zeros_scales, N, group_size, SQ_ALGO_AUTO);
}

// I W_hat^T + R in one launch; R [bs, seq, N] fp16.  Call shape of the fused variant the
// reference's kernel test imports (reference: quantization/nvidia/script/gemm_awq_test.py:63-65).
at::Tensor gemm_awq_residual_ut(at::Tensor I, at::Tensor W, at::Tensor W_zeros_scales, at::Tensor R, const int M,
                                const int N, const int K, const int group_size) {
    (void)M;
    (void)K;
    return gemm_impl(I, W, W_zeros_scales, N, group_size, SQ_ALGO_AUTO, c10::nullopt, R, SQ_ACT_NONE);
}

int act_code(const std::string& act) {
    if (act == "relu") return SQ_ACT_RELU;
    if (act == "silu") return SQ_ACT_SILU;
    if (act != "none" && !act.empty()) throw std::invalid_argument("unknown activation: " + act);
    return SQ_ACT_NONE;
}

// act(I W_hat^T + bias) + residual in one launch; bias [N] / residual [bs, seq, N] optional,
// act "none", "relu" or "silu".
at::Tensor gemm_awq_fused_ut(at::Tensor I, at::Tensor W, at::Tensor W_zeros_scales, c10::optional<at::Tensor> bias,
                             c10::optional<at::Tensor> residual, const std::string& act, const int N,
                             const int group_size) {
    return gemm_impl(I, W, W_zeros_scales, N, group_size, SQ_ALGO_AUTO, bias, residual, act_code(act));
}

// silu(I W1_hat^T) * (I W2_hat^T), [bs, seq, N].  Either the two weights with their zeros_scales, or one packed
// weight cat(W1, W2) along the output dimension (2N outputs) with its zeros_scales; the others None.  Argument
// order of the fused variant the reference's kernel test imports, which is also where the expected value comes
// from (reference: quantization/nvidia/script/gemm_awq_test.py:50-56,66-72).
at::Tensor gemm_awq_silu_dot_ut(at::Tensor I, c10::optional<at::Tensor> W1, c10::optional<at::Tensor> W2,
                                c10::optional<at::Tensor> ZS1, c10::optional<at::Tensor> ZS2,
                                c10::optional<at::Tensor> W13, c10::optional<at::Tensor> ZS13, const int M, const int N,
                                const int K, const int group_size) {
    (void)M;
    (void)K;
    auto has = [](const c10::optional<at::Tensor>& t) { return t.has_value() && t->defined(); };
    const bool packed = has(W13) && has(ZS13);
    if (!packed && !(has(W1) && has(W2) && has(ZS1) && has(ZS2)))
        throw std::invalid_argument("pass W1, W2 and their zeros_scales, or the packed weight and its zeros_scales");
    SQ_CHECK_DEVICE(I);
    SQ_CHECK_CONTIGUOUS(I);
    SQ_CHECK_DTYPE(I, at::kHalf);
    SQ_CHECK_DIMS(I, 3);
    const int64_t rows = I.size(0) * I.size(1);
    const int64_t Kin = I.size(2);
    if (group_size <= 0 || Kin % group_size != 0) throw std::invalid_argument("embbed dim must be a multiple of group_size!");
    TORCH_CHECK(rows < (1LL << 31) && Kin < (1LL << 31), "problem too large");
    c10::DeviceGuard guard(I.device());
    // Layout L1 views [N, K/2] / [N, 2K/g] of both halves (an int32-layout weight through the conversion cache).
    auto l1_of = [&](const at::Tensor& W, const at::Tensor& ZS, int n_out) {
        SQ_CHECK_DEVICE(W);
        SQ_CHECK_DEVICE(ZS);
        SQ_CHECK_CONTIGUOUS(W);
        SQ_CHECK_CONTIGUOUS(ZS);
        SQ_CHECK_DTYPE(ZS, at::kHalf);
        SQ_CHECK_DIMS(W, 2);
        SQ_CHECK_DIMS(ZS, 2);
        if (layout_of(W) == SQ_LAYOUT_L1) {
            if (W.size(0) != n_out) throw std::invalid_argument("output dim mismatch!");
            if (W.size(1) * 2 != Kin) throw std::invalid_argument("input dim mismatch!");
            if (ZS.size(0) != n_out || ZS.size(1) != 2 * (Kin / group_size))
                throw std::invalid_argument("zeros_scales shape mismatch!");
            return std::make_pair(W, ZS);
        }
        if (W.size(0) != Kin) throw std::invalid_argument("input dim mismatch!");
        if (W.size(1) * 8 != n_out) throw std::invalid_argument("output dim mismatch!");
        if (group_size != 128) throw std::runtime_error("unsupported group size");
        if (ZS.size(0) != Kin / group_size || ZS.size(1) != 2 * (int64_t)n_out)
            throw std::invalid_argument("zeros_scales shape mismatch!");
        return l1_view_of_l2(W, ZS, n_out, (int)Kin, group_size);
    };
    std::pair<at::Tensor, at::Tensor> gate, up;
    if (packed) {
        const auto both = l1_of(*W13, *ZS13, 2 * N);
        gate = {both.first.narrow(0, 0, N), both.second.narrow(0, 0, N)};
        up = {both.first.narrow(0, N, N), both.second.narrow(0, N, N)};
    } else {
        gate = l1_of(*W1, *ZS1, N);
        up = l1_of(*W2, *ZS2, N);
    }
    at::Tensor O = torch::empty({I.size(0), I.size(1), N}, I.options());
    at::Tensor up_out = torch::empty({rows, (int64_t)N}, I.options());
    void* stream = current_stream(I);
    void* ws_ptr = nullptr;
    size_t ws_bytes = 0;
    at::Tensor ws;
    if (rows > 2 && rows <= 1024) {
        ws = workspace_for(I, stream, sq_w4a16_workspace_bytes((int)rows, N, (int)Kin));
        ws_ptr = ws.data_ptr();
        ws_bytes = (size_t)ws.numel();
    }
    raise_if_error(sq_w4a16_gemm_silu_dot(I.data_ptr(), gate.first.data_ptr(), gate.second.data_ptr(),
                                          up.first.data_ptr(), up.second.data_ptr(), O.data_ptr(), up_out.data_ptr(),
                                          (int)rows, N, (int)Kin, group_size, SQ_LAYOUT_L1, ws_ptr, ws_bytes, stream),
                   "gemm_awq_silu_dot_ut");
    return O;
}

// act(LayerNorm(I) W_hat^T + bias) + residual: the pre-LN pattern of a decoder layer (nn.LayerNorm followed by
// the linear).  With up to 8 tokens, group size 128 and 2048 < K <= 4096 the normalisation happens inside the
// linear's kernel; otherwise a LayerNorm launch into a temporary comes first.
at::Tensor gemm_awq_ln_fused_ut(at::Tensor I, c10::optional<at::Tensor> ln_weight, c10::optional<at::Tensor> ln_bias,
                                double ln_eps, at::Tensor W, at::Tensor W_zeros_scales, c10::optional<at::Tensor> bias,
                                c10::optional<at::Tensor> residual, const std::string& act, const int N,
                                const int group_size) {
    const LnArgs ln{ln_weight, ln_bias, ln_eps};
    return gemm_impl(I, W, W_zeros_scales, N, group_size, SQ_ALGO_AUTO, bias, residual, act_code(act), &ln);
}

// Same with an explicit kernel id (SQ_ALGO_* | tuning word << 8); for tests and benchmarks.
at::Tensor gemm_awq_algo(at::Tensor I, at::Tensor W, at::Tensor W_zeros_scales, const int N, const int group_size,
                         const int algo) {
    return gemm_impl(I, W, W_zeros_scales, N, group_size, algo);
}

at::Tensor dequant(at::Tensor W, at::Tensor zeros_scales, const int N, const int K, const int group_size) {
    SQ_CHECK_DEVICE(W);
    SQ_CHECK_DEVICE(zeros_scales);
    SQ_CHECK_CONTIGUOUS(W);
    SQ_CHECK_CONTIGUOUS(zeros_scales);
    SQ_CHECK_DTYPE(zeros_scales, at::kHalf);
    SQ_CHECK_DIMS(W, 2);
    const int layout = layout_of(W);
    if (layout == SQ_LAYOUT_L1) {
        if (W.size(0) != N || W.size(1) * 2 != K) throw std::invalid_argument("weight shape mismatch!");
    } else {
        if (W.size(0) != K || W.size(1) * 8 != N) throw std::invalid_argument("weight shape mismatch!");
    }
    if (group_size <= 0 || K % group_size != 0 || zeros_scales.numel() != 2 * (int64_t)N * (K / group_size))
        throw std::invalid_argument("zeros_scales shape mismatch!");
    c10::DeviceGuard guard(W.device());
    at::Tensor out = torch::empty({N, K}, zeros_scales.options());
    raise_if_error(sq_w4a16_dequant(W.data_ptr(), zeros_scales.data_ptr(), out.data_ptr(), N, K, group_size, layout,
                                    current_stream(W)),
                   "dequant");
    return out;
}

void transpose_merge_zeros_scales(at::Tensor zeros, at::Tensor scales, at::Tensor zeros_scales, int in_features,
                                  int out_features, int group_size) {
    SQ_CHECK_DEVICE(zeros);
    SQ_CHECK_DEVICE(scales);
    SQ_CHECK_DEVICE(zeros_scales);
    SQ_CHECK_CONTIGUOUS(zeros);
    SQ_CHECK_CONTIGUOUS(scales);
    SQ_CHECK_CONTIGUOUS(zeros_scales);
    SQ_CHECK_DTYPE(zeros, at::kHalf);
    SQ_CHECK_DTYPE(scales, at::kHalf);
    SQ_CHECK_DTYPE(zeros_scales, at::kHalf);
    TORCH_CHECK(group_size > 0 && in_features % group_size == 0, "in_features must be a multiple of group_size");
    const int64_t count = (int64_t)out_features * (in_features / group_size);
    TORCH_CHECK(zeros.numel() == count && scales.numel() == count && zeros_scales.numel() == 2 * count,
                "zeros / scales / zeros_scales sizes do not match in_features, out_features, group_size");
    c10::DeviceGuard guard(zeros.device());
    raise_if_error(sq_transpose_merge_zeros_scales(zeros.data_ptr(), scales.data_ptr(), zeros_scales.data_ptr(),
                                                   in_features, out_features, group_size, current_stream(zeros)),
                   "transpose_merge_zeros_scales");
}

void convert_ours_to_awq(at::Tensor qweight_src, at::Tensor qweight_dst, int in_features, int out_features) {
    SQ_CHECK_DEVICE(qweight_src);
    SQ_CHECK_DEVICE(qweight_dst);
    SQ_CHECK_CONTIGUOUS(qweight_src);
    SQ_CHECK_CONTIGUOUS(qweight_dst);
    SQ_CHECK_DTYPE(qweight_src, at::kByte);
    TORCH_CHECK(qweight_src.numel() == (int64_t)out_features * in_features / 2, "qweight_src size mismatch");
    TORCH_CHECK((int64_t)qweight_dst.numel() * qweight_dst.element_size() == (int64_t)in_features * out_features / 2,
                "qweight_dst size mismatch");
    c10::DeviceGuard guard(qweight_src.device());
    raise_if_error(sq_convert_ours_to_awq(qweight_src.data_ptr(), qweight_dst.data_ptr(), in_features, out_features,
                                          current_stream(qweight_src)),
                   "convert_ours_to_awq");
}

void convert_awq_to_lmdeploy(at::Tensor qweight, at::Tensor qweight_dst, int in_features, int out_features) {
    SQ_CHECK_DEVICE(qweight);
    SQ_CHECK_DEVICE(qweight_dst);
    SQ_CHECK_CONTIGUOUS(qweight);
    SQ_CHECK_CONTIGUOUS(qweight_dst);
    SQ_CHECK_DTYPE(qweight_dst, at::kInt);
    TORCH_CHECK((int64_t)qweight.numel() * qweight.element_size() == (int64_t)in_features * out_features / 2,
                "qweight size mismatch");
    TORCH_CHECK(qweight_dst.numel() == (int64_t)in_features * out_features / 8, "qweight_dst size mismatch");
    c10::DeviceGuard guard(qweight.device());
    raise_if_error(sq_convert_awq_to_lmdeploy(qweight.data_ptr(), qweight_dst.data_ptr(), in_features, out_features,
                                              current_stream(qweight)),
                   "convert_awq_to_lmdeploy");
}

// 2-bit storage -> the 4-bit words the GEMM reads.  uint8 [N, K/4] -> uint8 [N, K/2] in layout L1;
// int32 [K, N/16] -> int32 [K, N/8] in layout L2 (there with the reference's own word arithmetic).
at::Tensor convert_2bit_to_4bit(at::Tensor qweight_2bit) {
    SQ_CHECK_DEVICE(qweight_2bit);
    SQ_CHECK_CONTIGUOUS(qweight_2bit);
    SQ_CHECK_DIMS(qweight_2bit, 2);
    TORCH_CHECK(qweight_2bit.dtype() == at::kByte || qweight_2bit.dtype() == at::kInt,
                "Tensor qweight_2bit must have dtype uint8 (layout L1) or int32 (layout L2)");
    c10::DeviceGuard guard(qweight_2bit.device());
    if (qweight_2bit.dtype() == at::kInt) {
        const int K = (int)qweight_2bit.size(0);
        const int N = (int)qweight_2bit.size(1) * 16;
        at::Tensor out = torch::empty({K, N / 8}, qweight_2bit.options());
        raise_if_error(
            sq_l2_convert_2bit_to_4bit(qweight_2bit.data_ptr(), out.data_ptr(), K, N, current_stream(qweight_2bit)),
            "convert_2bit_to_4bit");
        return out;
    }
    const int N = (int)qweight_2bit.size(0);
    const int K = (int)qweight_2bit.size(1) * 4;
    at::Tensor out = torch::empty({N, K / 2}, qweight_2bit.options());
    raise_if_error(sq_convert_2bit_to_4bit(qweight_2bit.data_ptr(), out.data_ptr(), N, K, current_stream(qweight_2bit)),
                   "convert_2bit_to_4bit");
    return out;
}

// int32 [K, N/8] -> int32 [K, N/16] (layout L2, the reference's word arithmetic).
at::Tensor convert_4bit_to_2bit(at::Tensor qweight_4bit) {
    SQ_CHECK_DEVICE(qweight_4bit);
    SQ_CHECK_CONTIGUOUS(qweight_4bit);
    SQ_CHECK_DTYPE(qweight_4bit, at::kInt);
    SQ_CHECK_DIMS(qweight_4bit, 2);
    TORCH_CHECK(qweight_4bit.size(1) % 2 == 0, "qweight_4bit needs an even number of words per row");
    c10::DeviceGuard guard(qweight_4bit.device());
    const int K = (int)qweight_4bit.size(0);
    const int N = (int)qweight_4bit.size(1) * 8;
    at::Tensor out = torch::empty({K, N / 16}, qweight_4bit.options());
    raise_if_error(
        sq_l2_convert_4bit_to_2bit(qweight_4bit.data_ptr(), out.data_ptr(), K, N, current_stream(qweight_4bit)),
        "convert_4bit_to_2bit");
    return out;
}

void clear_repack_cache() {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    for (auto& kv : g_repack_cache) drop_entry(kv.second);
    g_repack_cache.clear();
}

int repack_cache_size() {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    sweep_cache_locked();
    return (int)g_repack_cache.size();
}

}  // namespace

PYBIND11_MODULE(quant, m) {
    m.doc() = "W4A16 quantized linear for MI355X (gfx950): drop-in for the reference's `quant` extension";
    m.def("gemm_awq_ut", &gemm_awq_ut);
    m.def("dequant", &dequant);
    m.def("transpose_merge_zeros_scales", &transpose_merge_zeros_scales);
    m.def("convert_ours_to_awq", &convert_ours_to_awq);
    m.def("convert_awq_to_lmdeploy", &convert_awq_to_lmdeploy);
    // Additions without a counterpart in the reference's module.
    m.def("gemm_awq_algo", &gemm_awq_algo);
    m.def("gemm_awq_residual_ut", &gemm_awq_residual_ut);
    m.def("gemm_awq_fused_ut", &gemm_awq_fused_ut, py::arg("I"), py::arg("W"), py::arg("W_zeros_scales"),
          py::arg("bias") = py::none(), py::arg("residual") = py::none(), py::arg("act") = "none", py::arg("N"),
          py::arg("group_size"));
    m.def("gemm_awq_ln_fused_ut", &gemm_awq_ln_fused_ut, py::arg("I"), py::arg("ln_weight") = py::none(),
          py::arg("ln_bias") = py::none(), py::arg("ln_eps") = 1e-5, py::arg("W"), py::arg("W_zeros_scales"),
          py::arg("bias") = py::none(), py::arg("residual") = py::none(), py::arg("act") = "none", py::arg("N"),
          py::arg("group_size"));
    m.def("gemm_awq_silu_dot_ut", &gemm_awq_silu_dot_ut, py::arg("I"), py::arg("W1") = py::none(),
          py::arg("W2") = py::none(), py::arg("ZS1") = py::none(), py::arg("ZS2") = py::none(),
          py::arg("W13") = py::none(), py::arg("ZS13") = py::none(), py::arg("M"), py::arg("N"), py::arg("K"),
          py::arg("group_size"));
    m.def("convert_2bit_to_4bit", &convert_2bit_to_4bit);
    m.def("convert_4bit_to_2bit", &convert_4bit_to_2bit);
    m.def("clear_repack_cache", &clear_repack_cache);
    m.def("repack_cache_size", &repack_cache_size);
    m.def("version", []() { return sq_version(); });
}
