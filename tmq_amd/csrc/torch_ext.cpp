// PyTorch extension over the C ABI of include/tmq_hip.h: the reference's twelve binding names
// (tmq/tmq_cuda.cu:800-809, tmq/tmq_native.cpp:550-555) with the same argument order, so that
// `from .tmq_cuda import ...` / `from .tmq_native import ...` in tmq/tmq.py:28-46 can be pointed at this
// module unchanged. It only marshals: contiguity, device guard, current stream, output allocation,
// status -> exception. No kernel lives here. (PyTorch on ROCm presents the GPU as device type "cuda":
// the generic DeviceGuard resolves to the right implementation.)
//
// Built by `make -C tmq_amd/csrc ext` (g++, links libtmq_hip.so) into tmq_amd/tmq_hip_ext*.so.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>

#include <list>
#include <map>
#include <mutex>
#include <stdexcept>
#include <utility>
#include <vector>

#include "tmq_hip.h"

namespace {

void check(int rc, const char *what) {
    TORCH_CHECK(rc == TMQ_OK, what, ": ", tmq_status_string(rc),
                rc == TMQ_ERR_LAUNCH ? " (hipError " + std::to_string(tmq_last_hip_error()) + ")" : std::string());
}

void *stream_of(const torch::Tensor &t) { return at::hip::getCurrentHIPStream(t.device().index()).stream(); }

// Checks of the reference's soft-step hosts (tmq/tmq_cuda.cu:690-794): GPU tensor; fp16 is "not
// implemented yet" there (std::invalid_argument -> ValueError) and stays so.
torch::Tensor f32_cuda(const torch::Tensor &t, const char *name) {
    TORCH_CHECK(t.device().is_cuda(), name, ": expected a tensor on the GPU");
    if (t.scalar_type() == torch::kFloat16) throw std::invalid_argument("Not implemented yet");
    TORCH_CHECK(t.scalar_type() == torch::kFloat32, "Expected either a float16 or a float32 tensor as input/output");
    return t.contiguous();
}

torch::Tensor fwd_softstep(torch::Tensor weights, double digamma) {   // tmq_cuda.cu:740-764
    auto w = f32_cuda(weights, "fwd_softstep");
    const c10::DeviceGuard guard(w.device());
    auto y = torch::empty_like(w);
    check(tmq_softstep_fwd(w.data_ptr<float>(), y.data_ptr<float>(), w.numel(), digamma, stream_of(w)), "fwd_softstep");
    return y;
}

torch::Tensor bwd_softstep(torch::Tensor weights, double digamma, double scale, torch::Tensor grad) {   // 768-794
    auto w = f32_cuda(weights, "bwd_softstep"), g = f32_cuda(grad, "bwd_softstep");
    TORCH_CHECK(w.numel() == g.numel(), "bwd_softstep: weights and gradient differ in size");
    const c10::DeviceGuard guard(w.device());
    auto y = torch::empty_like(w);
    check(tmq_softstep_bwd(w.data_ptr<float>(), g.data_ptr<float>(), y.data_ptr<float>(), w.numel(), digamma, scale,
                           stream_of(w)), "bwd_softstep");
    return y;
}

torch::Tensor fwd_softstep_derivative(torch::Tensor weights, double digamma, double strength) {   // 690-709
    auto w = f32_cuda(weights, "fwd_softstep_derivative");
    const c10::DeviceGuard guard(w.device());
    auto y = torch::empty_like(w);
    check(tmq_softstep_deriv_fwd(w.data_ptr<float>(), y.data_ptr<float>(), w.numel(), digamma, strength, stream_of(w)),
          "fwd_softstep_derivative");
    return y;
}

torch::Tensor bwd_softstep_derivative(torch::Tensor weights, double digamma, double scale, torch::Tensor grad) {   // 713-735
    auto w = f32_cuda(weights, "bwd_softstep_derivative"), g = f32_cuda(grad, "bwd_softstep_derivative");
    TORCH_CHECK(w.numel() == g.numel(), "bwd_softstep_derivative: weights and gradient differ in size");
    const c10::DeviceGuard guard(w.device());
    auto y = torch::empty_like(w);
    check(tmq_softstep_deriv_bwd(w.data_ptr<float>(), g.data_ptr<float>(), y.data_ptr<float>(), w.numel(), digamma,
                                 scale, stream_of(w)), "bwd_softstep_derivative");
    return y;
}

// ---- one launch for all layers of a training step -------------------------------------------------
// Additive (no counterpart among the reference's bindings): SoftStep.forward / backward of every layer
// (tmq/tmq.py:404-438), the quantization loss (298-310) and its gradient (475-493) as multi-tensor
// launches. Outputs are carved from one flat buffer per call, each on a 256-byte boundary.
struct Carved {
    torch::Tensor flat;
    std::vector<torch::Tensor> parts;
};

Carved carve(const std::vector<torch::Tensor> &like) {
    int64_t total = 0;
    std::vector<int64_t> offs;
    for (const auto &t : like) {
        offs.push_back(total);
        total += (t.numel() + 63) / 64 * 64;
    }
    Carved c;
    c.flat = torch::empty({total}, like[0].options());
    for (size_t i = 0; i < like.size(); i++) {
        auto part = torch::empty({0}, like[0].options());
        part.set_(c.flat.storage(), offs[i], like[i].sizes(), like[i].strides());
        c.parts.push_back(part);
    }
    return c;
}

std::vector<torch::Tensor> step_weights(const std::vector<torch::Tensor> &weights, const char *name) {
    TORCH_CHECK(!weights.empty(), name, ": no tensors");
    std::vector<torch::Tensor> ws;
    for (const auto &w : weights) {
        ws.push_back(f32_cuda(w.detach(), name));
        TORCH_CHECK(ws.back().device() == ws[0].device(), name, ": all tensors must live on one device");
    }
    return ws;
}

// The accumulator cells of the loss reductions that finish inside their launch: one zero-filled buffer per device
// and stream, made on first use; every launch leaves it zero.
torch::Tensor loss_state(const torch::Tensor &like) {
    static std::mutex guard;
    static std::map<std::pair<int, void *>, torch::Tensor> states;
    const auto key = std::make_pair((int)like.device().index(), stream_of(like));
    std::lock_guard<std::mutex> lock(guard);
    auto it = states.find(key);
    if (it == states.end())
        it = states.emplace(key, torch::zeros({(int64_t)tmq_loss_state_bytes()}, like.options().dtype(torch::kUInt8))).first;
    return it->second;
}

std::tuple<std::vector<torch::Tensor>, c10::optional<torch::Tensor>> softstep_fwd_all(
        std::vector<torch::Tensor> weights, double digamma, bool want_loss, double sharpness, double strength) {
    auto ws = step_weights(weights, "softstep_fwd_all");
    const c10::DeviceGuard guard(ws[0].device());
    Carved ys = carve(ws);
    std::vector<tmq_step_tensor> table(ws.size());
    for (size_t i = 0; i < ws.size(); i++)
        table[i] = tmq_step_tensor{ws[i].data_ptr<float>(), nullptr, ys.parts[i].data_ptr<float>(), (uint64_t)ws[i].numel()};
    c10::optional<torch::Tensor> loss;
    torch::Tensor workspace;
    if (want_loss) {
        loss = torch::empty({}, ws[0].options());
        // finished inside the launch where the shape allows (up to 64 tensors of up to 2^18 blocks each)
        auto state = loss_state(ws[0]);
        const int status = tmq_softstep_fwd_multi_inlaunch(table.data(), (int)table.size(), digamma, sharpness, strength,
                                                           nullptr, loss->data_ptr<float>(), state.data_ptr(), stream_of(ws[0]));
        if (status != TMQ_ERR_UNSUPPORTED) {
            check(status, "softstep_fwd_all");
            return {ys.parts, loss};
        }
        workspace = torch::empty({(int64_t)tmq_softstep_multi_workspace_bytes(table.data(), (int)table.size())},
                                 ws[0].options().dtype(torch::kUInt8));
    }
    check(tmq_softstep_fwd_multi(table.data(), (int)table.size(), digamma, sharpness, strength, nullptr,
                                 want_loss ? loss->data_ptr<float>() : nullptr, want_loss ? workspace.data_ptr() : nullptr,
                                 stream_of(ws[0])), "softstep_fwd_all");
    return {ys.parts, loss};
}

std::vector<c10::optional<torch::Tensor>> softstep_bwd_all(std::vector<torch::Tensor> weights,
                                                           std::vector<c10::optional<torch::Tensor>> grads,
                                                           c10::optional<torch::Tensor> loss_upstream, double digamma,
                                                           double sharpness, double strength) {
    auto ws = step_weights(weights, "softstep_bwd_all");
    TORCH_CHECK(grads.size() == ws.size(), "softstep_bwd_all: one gradient (or None) per tensor");
    const c10::DeviceGuard guard(ws[0].device());
    torch::Tensor up;
    if (loss_upstream.has_value()) {
        TORCH_CHECK(loss_upstream->device().is_cuda() && loss_upstream->numel() == 1,
                    "softstep_bwd_all: loss_upstream must be one value on the GPU");
        up = loss_upstream->detach().to(torch::kFloat32).contiguous();
    }
    std::vector<size_t> live;
    std::vector<torch::Tensor> like, gs;
    for (size_t i = 0; i < ws.size(); i++)
        if (grads[i].has_value() || up.defined()) {
            live.push_back(i);
            like.push_back(ws[i]);
        }
    std::vector<c10::optional<torch::Tensor>> out(ws.size());
    if (live.empty()) return out;
    Carved dws = carve(like);
    std::vector<tmq_step_tensor> table(live.size());
    for (size_t k = 0; k < live.size(); k++) {
        const size_t i = live[k];
        const float *gp = nullptr;
        if (grads[i].has_value()) {
            const auto &g = *grads[i];
            TORCH_CHECK(g.device() == ws[i].device() && g.scalar_type() == torch::kFloat32 && g.numel() == ws[i].numel(),
                        "softstep_bwd_all: a gradient must match its weights in device, dtype and size");
            gs.push_back(g.detach().contiguous());
            gp = gs.back().data_ptr<float>();
        }
        table[k] = tmq_step_tensor{ws[i].data_ptr<float>(), gp, dws.parts[k].data_ptr<float>(), (uint64_t)ws[i].numel()};
        out[i] = dws.parts[k];
    }
    check(tmq_softstep_bwd_multi(table.data(), (int)table.size(), digamma, sharpness, strength,
                                 up.defined() ? up.data_ptr<float>() : nullptr, stream_of(ws[0])), "softstep_bwd_all");
    return out;
}

// ---- ternary inference -----------------------------------------------------------------------------
// The reference hands the compact words to every call; the kernels want the re-tiled layout, built
// once per weight tensor. A small LRU keeps (words -> native) pairs; an entry holds a reference to
// its words tensor, so the storage address it is keyed on cannot be recycled while it is cached.
struct NativeEntry {
    const void *ptr;
    int64_t version, K, Q, columns;
    torch::Tensor words, native;
};
std::list<NativeEntry> g_native;
std::mutex g_native_mutex;
constexpr size_t kNativeCacheSize = 64;

torch::Tensor native_of(const torch::Tensor &words, int64_t columns) {
    std::lock_guard<std::mutex> lock(g_native_mutex);
    const int64_t K = words.size(0), Q = words.size(1), version = words._version();
    for (auto it = g_native.begin(); it != g_native.end(); ++it)
        if (it->ptr == words.data_ptr() && it->version == version && it->K == K && it->Q == Q &&
            it->columns == columns && it->words.device() == words.device()) {
            g_native.splice(g_native.begin(), g_native, it);
            return g_native.front().native;
        }
    auto native = torch::empty({(int64_t)tmq_native_weight_bytes(columns, K)},
                               torch::dtype(torch::kUInt8).device(words.device()));
    check(tmq_prepack_weights(reinterpret_cast<const uint32_t *>(words.data_ptr<int32_t>()), columns, K, 1, 1,
                              native.data_ptr(), stream_of(words)), "prepack_weights");
    g_native.push_front(NativeEntry{words.data_ptr(), version, K, Q, columns, words, native});
    if (g_native.size() > kNativeCacheSize) g_native.pop_back();
    return native;
}

void check_mm_args(const torch::Tensor &lhs, const torch::Tensor &weights, int64_t columns, const char *name) {
    // tmq/tmq_cuda.cu:480-490, 566-575
    TORCH_CHECK(lhs.device().is_cuda() && weights.device().is_cuda(), name, ": expected tensors on the GPU");
    TORCH_CHECK(lhs.scalar_type() == torch::kFloat32 || lhs.scalar_type() == torch::kFloat16, name,
                ": expected fp32 (or fp16) activations");
    TORCH_CHECK(weights.dim() == 2 && weights.scalar_type() == torch::kInt32, name, ": expected 2-D int32 compact weights");
    TORCH_CHECK(weights.size(1) * 16 >= columns && weights.size(1) * 16 < columns + 16, name,
                ": compact weight width does not match the number of columns");
}

// fp32 activations (the reference's convention). The kernels carry them as fp16 terms, so the tensor is first
// scaled by the power of two that brings its largest value into fp16's range (tmq_f32_prescale; exact, undone
// in the epilogue's per-channel scale): any magnitude works, as with the reference's fp32 arithmetic. Many
// The two terms travel as row pairs of one fp16 pass wherever tmq_ternary_linear_ws takes the shape; otherwise many
// rows run the fp16 kernels over the two fp16 terms, y = W hi + W lo, and few rows the kernels that split on the fly.
torch::Tensor linear_f32(const torch::Tensor &x, int64_t M, int64_t K, const torch::Tensor &native, int64_t columns,
                         torch::Tensor &y, const char *name) {
    if (tmq_fp32_rows_self_scaled_for(x.data_ptr(), M, K, columns)) {   // one row (two over a small layer) the kernel scales itself: one launch
        check(tmq_ternary_linear(x.data_ptr(), TMQ_F32, M, K, native.data_ptr(), columns, nullptr, y.data_ptr(), stream_of(x)), name);
        return y;
    }
    // fp16 row pairs made once in a workspace, one pass of the fp16 kernels with the pairs added in the epilogue
    // (tmq_ternary_linear_ws: two or more rows over whole 64-index tiles)
    if (const size_t pairs = tmq_ternary_linear_workspace_bytes(TMQ_F32, M, K, columns);
        pairs && reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0) {
        auto ws = torch::empty({(int64_t)pairs}, x.options().dtype(torch::kUInt8));
        check(tmq_ternary_linear_ws(x.data_ptr(), TMQ_F32, M, K, native.data_ptr(), columns, nullptr, y.data_ptr(), ws.data_ptr(),
                                    pairs, stream_of(x)), name);
        return y;
    }
    const bool two_pass = tmq_fp32_rows_prefer_split(M, K, columns) != 0;
    auto fopt = x.options().dtype(torch::kFloat32);
    auto prescale = torch::empty({2}, fopt), scale = torch::empty({columns}, fopt);
    torch::Tensor xs, workspace;
    if (!two_pass) xs = torch::empty_like(x);
    const size_t wsb = tmq_f32_prescale_workspace_bytes(x.numel());
    if (wsb) workspace = torch::empty({(int64_t)wsb}, x.options().dtype(torch::kUInt8));
    check(tmq_f32_prescale(x.data_ptr<float>(), x.numel(), prescale.data_ptr<float>(), two_pass ? nullptr : xs.data_ptr<float>(),
                           nullptr, scale.data_ptr<float>(), columns, wsb ? workspace.data_ptr() : nullptr, stream_of(x)), name);
    if (!two_pass) {
        tmq_epilogue ep = {scale.data_ptr<float>(), nullptr, nullptr, 0, TMQ_F32};
        check(tmq_ternary_linear(xs.data_ptr(), TMQ_F32, M, K, native.data_ptr(), columns, &ep, y.data_ptr(), stream_of(x)), name);
        return y;
    }
    auto hi = torch::empty_like(x, x.options().dtype(torch::kFloat16));
    auto lo = torch::empty_like(hi);
    check(tmq_split_f32_scaled(x.data_ptr<float>(), prescale.data_ptr<float>(), hi.data_ptr(), lo.data_ptr(), x.numel(),
                               stream_of(x)), name);
    auto t = torch::empty_like(y);
    tmq_epilogue ep1 = {scale.data_ptr<float>(), nullptr, nullptr, 0, TMQ_F32};
    check(tmq_ternary_linear(hi.data_ptr(), TMQ_F16, M, K, native.data_ptr(), columns, &ep1, t.data_ptr(), stream_of(x)), name);
    tmq_epilogue ep2 = {scale.data_ptr<float>(), nullptr, t.data_ptr(), 0, TMQ_F32};
    check(tmq_ternary_linear(lo.data_ptr(), TMQ_F16, M, K, native.data_ptr(), columns, &ep2, y.data_ptr(), stream_of(x)), name);
    return y;
}

torch::Tensor ternary_mmm_cuda(torch::Tensor lhs, torch::Tensor weights, int64_t columns) {   // tmq_cuda.cu:478-549
    check_mm_args(lhs, weights, columns, "ternary_mmm_cuda");
    TORCH_CHECK(lhs.dim() >= 1 && lhs.dim() <= 4, "ternary_mmm_cuda: expected 1 to 4 dimensions");
    const int64_t K = weights.size(0);
    TORCH_CHECK(lhs.size(-1) == K, "ternary_mmm_cuda: the last dimension of the input must equal the weight rows");
    const c10::DeviceGuard guard(lhs.device());
    auto x = lhs.contiguous();
    auto w = weights.contiguous();
    auto native = native_of(w, columns);
    std::vector<int64_t> shape = lhs.dim() == 1 ? std::vector<int64_t>{1, columns} : lhs.sizes().vec();
    shape.back() = columns;
    auto y = torch::empty(shape, lhs.options().dtype(torch::kFloat32));
    const int64_t M = K ? x.numel() / K : 0;
    if (M == 0) return y;
    if (x.scalar_type() == torch::kFloat32) return linear_f32(x, M, K, native, columns, y, "ternary_mmm_cuda");
    // shapes that gain from a workspace (partial sums of a reduction cut across workgroups; a padded copy of rows
    // whose length is no multiple of 64) get one
    if (const size_t bytes = M > 16 && (M <= 32 || K % 64) ? tmq_ternary_linear_workspace_bytes(TMQ_F16, M, K, columns) : 0) {
        auto ws = torch::empty({(int64_t)bytes}, x.options().dtype(torch::kUInt8));
        check(tmq_ternary_linear_ws(x.data_ptr(), TMQ_F16, M, K, native.data_ptr(), columns, nullptr, y.data_ptr(), ws.data_ptr(),
                                    bytes, stream_of(x)), "ternary_mmm_cuda");
        return y;
    }
    check(tmq_ternary_linear(x.data_ptr(), TMQ_F16, M, K, native.data_ptr(), columns, nullptr, y.data_ptr(), stream_of(x)),
          "ternary_mmm_cuda");
    return y;
}

torch::Tensor ternary_mvm_cuda(torch::Tensor vector, torch::Tensor weights, int64_t columns) {   // tmq_cuda.cu:563-603
    check_mm_args(vector, weights, columns, "ternary_mvm_cuda");
    TORCH_CHECK(vector.dim() >= 1 && vector.dim() <= 4, "ternary_mvm_cuda: expected 1 to 4 dimensions");
    const int64_t K = weights.size(0);
    TORCH_CHECK(vector.numel() == K, "ternary_mvm_cuda: expected a single vector of the weight rows' length");  // :584
    const c10::DeviceGuard guard(vector.device());
    auto x = vector.contiguous();
    auto native = native_of(weights.contiguous(), columns);
    std::vector<int64_t> shape = vector.sizes().vec();
    shape.back() = columns;
    auto y = torch::empty(shape, vector.options().dtype(torch::kFloat32));
    if (x.scalar_type() == torch::kFloat32) return linear_f32(x, 1, K, native, columns, y, "ternary_mvm_cuda");
    check(tmq_ternary_linear(x.data_ptr(), TMQ_F16, 1, K, native.data_ptr(), columns, nullptr, y.data_ptr(), stream_of(x)),
          "ternary_mvm_cuda");
    return y;
}

// Depthwise convolution on the unfolded input (tmq/tmq_cuda.cu:607-642, caller tmq/tmq.py:849-853):
// in [..., positions, ky * kx * channels] (tap-major, channel fastest), weights = compact words of the
// [channels, 1, ky, kx] kernel; out [..., positions, channels], out[p][c] = sum_t in[p][t C + c] T[c][t].
torch::Tensor ternary_dwconv_cuda(torch::Tensor input, torch::Tensor weights, int64_t kx, int64_t ky, int64_t channels) {
    TORCH_CHECK(input.device().is_cuda() && weights.device().is_cuda(), "ternary_dwconv_cuda: expected tensors on the GPU");
    TORCH_CHECK(input.scalar_type() == torch::kFloat32 || input.scalar_type() == torch::kFloat16,
                "ternary_dwconv_cuda: expected fp32 (or fp16) input");
    const int64_t taps = kx * ky;
    TORCH_CHECK(weights.scalar_type() == torch::kInt32 && weights.numel() == taps * ((channels + 15) / 16),
                "ternary_dwconv_cuda: compact weights do not match kernel size and channels");
    TORCH_CHECK(input.dim() >= 2 && input.size(-1) == taps * channels,
                "ternary_dwconv_cuda: the last dimension must be ky * kx * channels");
    const c10::DeviceGuard guard(input.device());
    auto x = input.contiguous();
    auto w = weights.contiguous();
    std::vector<int64_t> shape = input.sizes().vec();
    shape.back() = channels;
    auto y = torch::empty(shape, input.options().dtype(torch::kFloat32));
    const int64_t P = x.numel() / (taps * channels);
    check(tmq_ternary_dwconv_patches(x.data_ptr(), x.scalar_type() == torch::kFloat16 ? TMQ_F16 : TMQ_F32, P, (int32_t)taps,
                                     channels, reinterpret_cast<const uint32_t *>(w.data_ptr<int32_t>()),
                                     y.data_ptr<float>(), stream_of(x)), "ternary_dwconv_cuda");
    return y;
}

// Transposed depthwise variant in column form (tmq/tmq_cuda.cu:645-686, caller tmq/tmq.py:1026-1029):
// in fp32 [P, C], [B, P, C] or [B, 1, P, C]; weights = compact words of the [C, 1, ky, kx] kernel shaped
// [1, *, *, ceil(C/16)]; out [.., C * taps, P], out[c taps + t][p] = in[p][c] T[c][t], ready for F.fold.
// Every batch entry is computed and a 4-D input gives the 4-D output (the reference's launch has no
// batch index and its 4-D result is overwritten by a 2-D one, tmq/tmq_cuda.cu:677-682).
torch::Tensor ternary_dwconvtrans_cuda(torch::Tensor input, torch::Tensor weights, int64_t kx, int64_t ky) {
    TORCH_CHECK(input.device().is_cuda() && weights.device().is_cuda(), "ternary_dwconvtrans_cuda: expected tensors on the GPU");
    TORCH_CHECK(input.scalar_type() == torch::kFloat32, "ternary_dwconvtrans_cuda: expected fp32 input");
    TORCH_CHECK(input.dim() >= 2 && input.dim() <= 4 && (input.dim() != 4 || input.size(1) == 1),
                "ternary_dwconvtrans_cuda: expected [P, C], [B, P, C] or [B, 1, P, C]");
    const int64_t taps = kx * ky, P = input.size(-2), C = input.size(-1), B = input.dim() > 2 ? input.size(0) : 1;
    TORCH_CHECK(weights.scalar_type() == torch::kInt32 && weights.dim() == 4 && weights.size(0) == 1 &&
                    weights.size(1) * weights.size(2) == taps && weights.size(3) == (C + 15) / 16,
                "ternary_dwconvtrans_cuda: compact weights do not match kernel size and channels");
    const c10::DeviceGuard guard(input.device());
    auto x = input.contiguous();
    auto w = weights.contiguous();
    std::vector<int64_t> shape = input.sizes().vec();
    shape[shape.size() - 2] = C * taps;
    shape.back() = P;
    auto y = torch::empty(shape, input.options());
    if (y.numel())
        check(tmq_ternary_dwconvtrans_cols(x.data_ptr<float>(), B, P, (int32_t)taps, C,
                                           reinterpret_cast<const uint32_t *>(w.data_ptr<int32_t>()), y.data_ptr<float>(),
                                           stream_of(x)), "ternary_dwconvtrans_cuda");
    return y;
}

// ---- pack / unpack / codec (tmq/tmq_native.cpp:418-544) -------------------------------------------------
torch::Device gpu_device() {
    TORCH_CHECK(at::cuda::is_available(), "tmq_hip_ext needs a GPU: its pack / unpack kernels have no CPU fallback");
    return torch::Device(torch::kCUDA, c10::hip::current_device());
}

int dtype_code(const torch::Tensor &t) {
    switch (t.scalar_type()) {
        case torch::kFloat32: return TMQ_F32;
        case torch::kInt32: return TMQ_I32;
        case torch::kInt8: return TMQ_I8;
        default: throw std::invalid_argument("Cannot handle the supplied data-type");   // tmq_native.cpp:292
    }
}

torch::Tensor compactify_ternary(torch::Tensor input) {   // tmq_native.cpp:418-425
    TORCH_CHECK(input.dim() == 2 || input.dim() == 4, "compactify_ternary: expected a tensor with 2 or 4 dimensions");
    const int code = dtype_code(input);
    const bool on_cpu = !input.device().is_cuda();
    auto src = (on_cpu ? input.to(gpu_device()) : input).contiguous();
    const c10::DeviceGuard guard(src.device());
    const int64_t N = src.size(0), K = N ? src.numel() / N : 0, Q = (N + 15) / 16;
    std::vector<int64_t> shape = src.dim() == 2 ? std::vector<int64_t>{src.size(1), Q}
                                                : std::vector<int64_t>{src.size(1), src.size(2), src.size(3), Q};
    auto out = torch::empty(shape, src.options().dtype(torch::kInt32));
    check(tmq_pack_ternary(src.data_ptr(), code, N, K, reinterpret_cast<uint32_t *>(out.data_ptr<int32_t>()),
                           stream_of(src)), "compactify_ternary");
    return on_cpu ? out.cpu() : out;
}

torch::Tensor decompress_ternary(torch::Tensor input, std::vector<int64_t> orig_shape) {   // tmq_native.cpp:489-503
    TORCH_CHECK(!input.device().is_cuda(), "decompress_ternary: expected a CPU tensor");
    TORCH_CHECK(input.dim() == 1 && input.scalar_type() == torch::kInt8 && input.numel() >= 26,
                "decompress_ternary: expected a 1-D int8 stream of at least 26 bytes");
    TORCH_CHECK(orig_shape.size() == 2 || orig_shape.size() == 4, "Shape needs to be of dim 2 or 4");
    const int64_t cols = orig_shape[0], qcols = (cols + 15) / 16;
    int64_t rows = 1;
    for (size_t i = 1; i < orig_shape.size(); i++) rows *= orig_shape[i];
    std::vector<int64_t> shape = orig_shape.size() == 4
        ? std::vector<int64_t>{orig_shape[1], orig_shape[2], orig_shape[3], qcols} : std::vector<int64_t>{rows, qcols};
    auto out = torch::empty(shape, torch::dtype(torch::kInt32));
    auto src = input.contiguous();
    check(tmq_decompress_ternary(reinterpret_cast<const uint8_t *>(src.data_ptr<int8_t>()), (size_t)src.numel(),
                                 reinterpret_cast<uint32_t *>(out.data_ptr<int32_t>()), rows, cols), "decompress_ternary");
    return out;
}

torch::Tensor expand_ternary(torch::Tensor input, std::vector<int64_t> orig_shape, bool entropy_decode) {   // 516-544
    if (entropy_decode) input = decompress_ternary(input, orig_shape);
    TORCH_CHECK(input.scalar_type() == torch::kInt32, "expand_ternary: expected an int32 tensor");
    if (orig_shape.size() != 2 && orig_shape.size() != 4) throw std::invalid_argument("Shape needs to be of dim 2 or 4");
    const bool on_cpu = !input.device().is_cuda();
    auto src = (on_cpu ? input.to(gpu_device()) : input).contiguous();
    const c10::DeviceGuard guard(src.device());
    const int64_t N = orig_shape[0];
    int64_t K = 1;
    for (size_t i = 1; i < orig_shape.size(); i++) K *= orig_shape[i];
    TORCH_CHECK(src.numel() == K * ((N + 15) / 16), "expand_ternary: packed tensor does not match the original shape");
    auto out = torch::empty(orig_shape, src.options().dtype(torch::kFloat32));
    check(tmq_unpack_ternary(reinterpret_cast<const uint32_t *>(src.data_ptr<int32_t>()), N, K, out.data_ptr<float>(),
                             stream_of(src)), "expand_ternary");
    return on_cpu ? out.cpu() : out;
}

torch::Tensor compress_ternary(torch::Tensor input, std::vector<int64_t> orig_shape, bool from_compact) {   // 439-477
    torch::Tensor words;
    if (from_compact) {
        TORCH_CHECK(input.scalar_type() == torch::kInt32 && (input.dim() == 2 || input.dim() == 4),
                    "compress_ternary: expected a 2-D or 4-D int32 compact tensor");
        words = input;
    } else {
        TORCH_CHECK(input.scalar_type() == torch::kFloat32, "compress_ternary: expected fp32 weights");
        words = compactify_ternary(input);
    }
    words = words.detach().cpu().contiguous();
    TORCH_CHECK(!orig_shape.empty(), "compress_ternary: empty shape");
    const int64_t columns = orig_shape[0], rows = words.numel() / ((columns + 15) / 16);
    const size_t cap = tmq_compress_bound(rows, columns);
    auto buf = torch::empty({(int64_t)cap}, torch::dtype(torch::kInt8));
    size_t size = 0;
    check(tmq_compress_ternary(reinterpret_cast<const uint32_t *>(words.data_ptr<int32_t>()), rows, columns,
                               reinterpret_cast<uint8_t *>(buf.data_ptr<int8_t>()), cap, &size), "compress_ternary");
    return buf.narrow(0, 0, (int64_t)size).clone();
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "TMQ hot path on MI355X: the reference's tmq_cuda / tmq_native bindings over libtmq_hip";
    // tmq_cuda (tmq/tmq_cuda.cu:800-809)
    m.def("fwd_softstep", &fwd_softstep);
    m.def("bwd_softstep", &bwd_softstep);
    m.def("fwd_softstep_derivative", &fwd_softstep_derivative);
    m.def("bwd_softstep_derivative", &bwd_softstep_derivative);
    m.def("ternary_mmm_cuda", &ternary_mmm_cuda);
    m.def("ternary_mvm_cuda", &ternary_mvm_cuda);
    m.def("ternary_dwconv_cuda", &ternary_dwconv_cuda);
    m.def("ternary_dwconvtrans_cuda", &ternary_dwconvtrans_cuda);
    // additive: all layers of a training step in one launch
    m.def("softstep_fwd_all", &softstep_fwd_all);
    m.def("softstep_bwd_all", &softstep_bwd_all);
    // tmq_native (tmq/tmq_native.cpp:550-555)
    m.def("compactify_ternary", &compactify_ternary);
    m.def("compress_ternary", &compress_ternary);
    m.def("decompress_ternary", &decompress_ternary);
    m.def("expand_ternary", &expand_ternary);
}
