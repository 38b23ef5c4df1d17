// Compiled host binding of libq4gptq for PyTorch-ROCm: the counterpart of the reference's pybind module
// (src/alpaca_lora_4bit/quant_cuda/quant_cuda.cpp:204-227), host code only (built by g++; the kernels live in
// libq4gptq.so behind the C ABI of include/q4_gptq.h).  Per call it does what the reference's binding leaves out
// -- dtype / shape / device / contiguity checks -- then takes torch's CURRENT stream for the tensors' device, finds
// the cached workspace of that (device, stream), allocates the output and calls q4_*.  Nothing here looks at tensor
// CONTENTS (whether g_idx is sequential, whether scales are small): the Python layer above decides that once per
// layer and passes g_idx = None for sequential groups.
#include <torch/extension.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>

#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "q4_gptq.h"

namespace py = pybind11;

namespace {

py::object g_error_class;      // alpaca_lora_4bit_amd._lib.Q4Error, set by Python at import

[[noreturn]] void raise_q4(int code, const char* what) {
    const std::string msg = std::string(what) + ": " + q4_error_string(code) + " (code " + std::to_string(code) + ")";
    if (g_error_class && !g_error_class.is_none()) {
        PyErr_SetString(g_error_class.ptr(), msg.c_str());
        throw py::error_already_set();
    }
    throw std::runtime_error(msg);
}

struct Layer {
    const int32_t* qweight;
    const int32_t* qzeros;
    const void* scales;
    const int32_t* g_idx;      // null: sequential groups
    int K, N, G, groupsize;
    c10::Device device;
};

// Shapes, dtypes, device and contiguity of a layer's tensors against each other (contents are not read).
Layer check_layer(const at::Tensor& qweight, const at::Tensor& qzeros, const at::Tensor& scales,
                  const c10::optional<at::Tensor>& g_idx, int64_t groupsize) {
    TORCH_CHECK_VALUE(qweight.is_cuda(), "qweight must be on the GPU");
    TORCH_CHECK_VALUE(qweight.scalar_type() == at::kInt && qweight.dim() == 2, "qweight must be int32 [K/8, N]");
    TORCH_CHECK_VALUE(qzeros.scalar_type() == at::kInt && qzeros.dim() == 2, "qzeros must be int32 [G, N/8]");
    TORCH_CHECK_VALUE(scales.scalar_type() == at::kHalf && scales.dim() == 2, "scales must be float16 [G, N]");
    const int64_t K = qweight.size(0) * 8, N = qweight.size(1), G = scales.size(0);
    TORCH_CHECK_VALUE(scales.size(1) == N && qzeros.size(0) == G && qzeros.size(1) == N / 8,
                      "scales / qzeros do not match qweight");
    const auto dev = qweight.device();
    TORCH_CHECK_VALUE(qweight.is_contiguous() && qzeros.is_contiguous() && scales.is_contiguous() &&
                      qzeros.device() == dev && scales.device() == dev,
                      "quantized tensors must be contiguous and on one device");
    TORCH_CHECK_VALUE(K < (1ll << 31) && N < (1ll << 31), "layer too large");
    const int32_t* gp = nullptr;
    if (g_idx.has_value()) {
        const at::Tensor& g = *g_idx;
        TORCH_CHECK_VALUE(g.scalar_type() == at::kInt && g.dim() == 1 && g.size(0) == K && g.is_contiguous() && g.device() == dev,
                          "g_idx must be a contiguous int32 [K] tensor on the same device");
        gp = g.data_ptr<int32_t>();
    } else {
        TORCH_CHECK_VALUE(groupsize > 0, "groupsize is required when g_idx is None");
    }
    return Layer{qweight.data_ptr<int32_t>(), qzeros.data_ptr<int32_t>(), scales.data_ptr(), gp,
                 (int)K, (int)N, (int)G, (int)groupsize, dev};
}

at::Tensor flat_half(const at::Tensor& x, int64_t cols, const c10::Device& dev, const char* what) {
    TORCH_CHECK_VALUE(x.is_cuda() && x.device() == dev, what, " must be on the layer's device");
    TORCH_CHECK_VALUE(x.dim() >= 1 && x.size(-1) == cols, what, " last dimension ", x.size(-1), " != ", cols);
    at::Tensor x2 = x.reshape({-1, cols});
    if (x2.scalar_type() != at::kHalf) x2 = x2.to(at::kHalf);
    return x2.contiguous();
}

std::vector<int64_t> out_sizes(const c10::optional<std::vector<int64_t>>& shape, int64_t rows, int64_t cols) {
    if (!shape.has_value()) return {rows, cols};
    int64_t n = 1;
    for (int64_t d : *shape) n *= d;
    TORCH_CHECK_VALUE(!shape->empty() && shape->back() == cols && n == rows * cols, "out_shape does not hold ", rows,
                      " rows of ", cols);
    return *shape;
}

// Per (device, stream) buffers.  `zeroed`: the GEMV's split-K accumulators, zero on first use and left zero by
// every completed call; `scratch`: partial sums whose contents never matter.
struct Buffers {
    at::Tensor zeroed, scratch;
};
std::mutex g_mutex;
std::map<std::pair<int, void*>, Buffers> g_buffers;
// A buffer that had to grow is kept, not freed: a HIP graph captured earlier still launches with the old pointer,
// and memory handed back to the caching allocator could by then belong to another tensor.
std::vector<at::Tensor> g_retired;
// Workspaces of the fused MLP step: one per (device, stream, M, H, I), because the hand-over words and the launch
// ticket they hold are only valid for calls of one shape.
struct MlpKey {
    int dev; void* stream; int M, H, I;
    bool operator<(const MlpKey& o) const {
        return std::tie(dev, stream, M, H, I) < std::tie(o.dev, o.stream, o.M, o.H, o.I);
    }
};
std::map<MlpKey, at::Tensor> g_mlp_buffers;
const bool g_check_workspace = [] { const char* e = getenv("Q4_CHECK_WORKSPACE"); return e && e[0] == '1'; }();

void* zeroed_workspace(const c10::Device& dev, void* stream, size_t nbytes, size_t* have) {
    std::lock_guard<std::mutex> lock(g_mutex);
    Buffers& b = g_buffers[{dev.index(), stream}];
    if (!b.zeroed.defined() || (size_t)b.zeroed.numel() < nbytes) {
        const int64_t n = (int64_t)std::max(nbytes, (size_t)1 << 22);
        if (b.zeroed.defined()) g_retired.push_back(b.zeroed);
        b.zeroed = at::zeros({n}, at::TensorOptions().dtype(at::kByte).device(dev));
    } else if (g_check_workspace) {
        // debugging aid: the invariant "every call leaves the accumulators zero" checked on entry (synchronises)
        if (b.zeroed.any().item<bool>()) {
            b.zeroed.zero_();
            TORCH_CHECK(false, "libq4gptq: the GEMV workspace of this stream was not zero on entry (an earlier call "
                               "was cut short, or two streams shared it); it has been cleared");
        }
    }
    *have = (size_t)b.zeroed.numel();
    return b.zeroed.data_ptr();
}

// A call that returned an error after (possibly) launching may have left partial sums behind: clear them, so
// that later products on this stream are not silently corrupted.
void reset_zeroed_workspace(const c10::Device& dev, void* stream) {
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_buffers.find({dev.index(), stream});
    if (it != g_buffers.end() && it->second.zeroed.defined()) it->second.zeroed.zero_();
}

void* scratch_workspace(const c10::Device& dev, void* stream, size_t nbytes, size_t* have) {
    *have = 0;
    if (nbytes == 0) return nullptr;
    std::lock_guard<std::mutex> lock(g_mutex);
    Buffers& b = g_buffers[{dev.index(), stream}];
    if (!b.scratch.defined() || (size_t)b.scratch.numel() < nbytes) {
        const int64_t n = (int64_t)std::max(nbytes, (size_t)1 << 22);
        if (b.scratch.defined()) g_retired.push_back(b.scratch);
        b.scratch = at::empty({n}, at::TensorOptions().dtype(at::kByte).device(dev));
    }
    *have = (size_t)b.scratch.numel();
    return b.scratch.data_ptr();
}

struct Launch {
    c10::hip::OptionalHIPGuard guard;
    void* stream;
    explicit Launch(const c10::Device& dev) {
        if (dev.index() != c10::hip::current_device()) guard.set_index(dev.index());
        stream = (void*)c10::hip::getCurrentHIPStream(dev.index()).stream();
    }
};

bool fill_drop(const c10::optional<std::pair<int64_t, double>>& dropout, q4_dropout_t* d) {
    if (!dropout.has_value() || dropout->second == 0.0) return false;
    TORCH_CHECK_VALUE(dropout->second >= 0.0 && dropout->second < 1.0, "dropout probability must be in [0, 1)");
    const uint64_t seed = (uint64_t)dropout->first;
    d->seed_lo = (uint32_t)(seed & 0xFFFFFFFFu);
    d->seed_hi = (uint32_t)(seed >> 32);
    d->p = (float)dropout->second;
    return true;
}

// ------------------------------------------------------------------------------------------------ operators
at::Tensor dequant(const at::Tensor& qweight, const at::Tensor& qzeros, const at::Tensor& scales,
                   const c10::optional<at::Tensor>& g_idx, int64_t groupsize, c10::optional<at::Tensor> out) {
    const Layer l = check_layer(qweight, qzeros, scales, g_idx, groupsize);
    at::Tensor o = out.has_value() ? *out : at::empty({l.K, l.N}, scales.options());
    TORCH_CHECK_VALUE(o.scalar_type() == at::kHalf && o.dim() == 2 && o.size(0) == l.K && o.size(1) == l.N && o.is_contiguous() &&
                      o.device() == l.device, "out must be a contiguous float16 [K, N] tensor on the same device");
    Launch L(l.device);
    const int rc = q4_dequant_f16(l.qweight, l.qzeros, l.scales, l.g_idx, l.groupsize, o.data_ptr(), l.K, l.N, l.G, L.stream);
    if (rc != Q4_OK) raise_q4(rc, "q4_dequant_f16");
    return o;
}

at::Tensor gemv(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& qzeros, const at::Tensor& scales,
                const c10::optional<at::Tensor>& g_idx, int64_t groupsize, c10::optional<at::Tensor> out, bool accumulate,
                const c10::optional<std::vector<int64_t>>& out_shape) {
    const Layer l = check_layer(qweight, qzeros, scales, g_idx, groupsize);
    const at::Tensor x2 = flat_half(x, l.K, l.device, "x");
    const int64_t M = x2.size(0);
    if (M == 0 && !out.has_value()) return at::empty(out_sizes(out_shape, 0, l.N), x2.options());
    TORCH_CHECK_VALUE(M >= 1 && M <= 16, "gemv handles 1..16 rows, got ", M);
    TORCH_CHECK_VALUE(out.has_value() || !accumulate, "accumulate needs an output tensor");
    at::Tensor o = out.has_value() ? *out : at::empty(out_sizes(out_shape, M, l.N), x2.options());
    TORCH_CHECK_VALUE(o.scalar_type() == at::kHalf && o.numel() == M * l.N && o.size(-1) == l.N && o.is_contiguous() &&
                      o.device() == l.device,
                      "out must be a contiguous float16 [..., N] tensor with M rows on the same device");
    Launch L(l.device);
    size_t have = 0;
    void* ws = zeroed_workspace(l.device, L.stream, q4_gemv_workspace_bytes((int)M, l.K, l.N), &have);
    const int rc = q4_gemv_f16(x2.data_ptr(), l.qweight, l.qzeros, l.scales, l.g_idx, l.groupsize, o.data_ptr(),
                               accumulate ? 1 : 0, (int)M, l.K, l.N, l.G, ws, have, L.stream);
    if (rc != Q4_OK) {
        if (rc == Q4_ERR_LAUNCH) reset_zeroed_workspace(l.device, L.stream);
        raise_q4(rc, "q4_gemv_f16");
    }
    return o;
}

// layers: list of (qweight, qzeros, scales); xs: one tensor per layer (the same tensor may repeat)
std::vector<at::Tensor> gemv_grouped(const std::vector<at::Tensor>& xs,
                                     const std::vector<std::tuple<at::Tensor, at::Tensor, at::Tensor>>& layers,
                                     int64_t groupsize, c10::optional<std::vector<at::Tensor>> outs, bool accumulate) {
    const size_t n = layers.size();
    TORCH_CHECK_VALUE(n >= 1 && n <= Q4_GEMV_MAX_GROUP, "gemv_grouped takes 1..", Q4_GEMV_MAX_GROUP, " layers");
    TORCH_CHECK_VALUE(xs.size() == n, "one activation tensor per layer");
    TORCH_CHECK_VALUE(!outs.has_value() || outs->size() == n, "one output per layer");
    TORCH_CHECK_VALUE(outs.has_value() || !accumulate, "accumulate needs output tensors");
    q4_gemv_layer_t desc[Q4_GEMV_MAX_GROUP];
    std::vector<at::Tensor> keep, result;
    int64_t M = -1, K = -1, total_n = 0;
    c10::optional<c10::Device> dev;
    for (size_t i = 0; i < n; ++i) {
        const Layer l = check_layer(std::get<0>(layers[i]), std::get<1>(layers[i]), std::get<2>(layers[i]), c10::nullopt, groupsize);
        if (!dev.has_value()) { dev = l.device; K = l.K; }
        TORCH_CHECK_VALUE(l.device == *dev && l.K == K, "grouped layers must share the device and K");
        at::Tensor x2;
        for (size_t j = 0; j < i; ++j)
            if (xs[j].is_same(xs[i])) { x2 = keep[j]; break; }
        if (!x2.defined()) x2 = flat_half(xs[i], K, *dev, "x");
        if (M < 0) M = x2.size(0);
        TORCH_CHECK_VALUE(x2.size(0) == M, "grouped layers must share the number of rows");
        keep.push_back(x2);
        desc[i].x = x2.data_ptr(); desc[i].qweight = l.qweight; desc[i].qzeros = l.qzeros; desc[i].scales = l.scales;
        desc[i].N = l.N;
        total_n += l.N;
    }
    TORCH_CHECK_VALUE(M >= 1 && M <= 16, "gemv handles 1..16 rows, got ", M);
    for (size_t i = 0; i < n; ++i) {
        at::Tensor o = outs.has_value() ? (*outs)[i] : at::empty({M, (int64_t)desc[i].N}, keep[i].options());
        TORCH_CHECK_VALUE(o.scalar_type() == at::kHalf && o.numel() == M * desc[i].N && o.size(-1) == desc[i].N &&
                          o.is_contiguous() && o.device() == *dev,
                          "outputs must be contiguous float16 [..., N_i] tensors with M rows on the same device");
        desc[i].y = o.data_ptr();
        result.push_back(o);
    }
    Launch L(*dev);
    size_t have = 0;
    void* ws = zeroed_workspace(*dev, L.stream, q4_gemv_grouped_workspace_bytes((int)M, (int)total_n), &have);
    const int rc = q4_gemv_grouped_f16(desc, (int)n, (int)groupsize, accumulate ? 1 : 0, (int)M, (int)K, ws, have, L.stream);
    if (rc != Q4_OK) {
        if (rc == Q4_ERR_LAUNCH) reset_zeroed_workspace(*dev, L.stream);
        raise_q4(rc, "q4_gemv_grouped_f16");
    }
    return result;
}

// y = down(silu(gate(x)) * up(x)) for 1..16 rows in one launch; each layer = (qweight, qzeros, scales), sequential groups.
// Returns y, or (y, gate_out, up_out) when `intermediates` is set.
std::vector<at::Tensor> mlp_decode(const at::Tensor& x, const std::tuple<at::Tensor, at::Tensor, at::Tensor>& gate,
                                   const std::tuple<at::Tensor, at::Tensor, at::Tensor>& up,
                                   const std::tuple<at::Tensor, at::Tensor, at::Tensor>& down, int64_t groupsize,
                                   bool intermediates, const c10::optional<std::vector<int64_t>>& out_shape) {
    const Layer lg = check_layer(std::get<0>(gate), std::get<1>(gate), std::get<2>(gate), c10::nullopt, groupsize);
    const Layer lu = check_layer(std::get<0>(up), std::get<1>(up), std::get<2>(up), c10::nullopt, groupsize);
    const Layer ld = check_layer(std::get<0>(down), std::get<1>(down), std::get<2>(down), c10::nullopt, groupsize);
    const int H = lg.K, I = lg.N;
    TORCH_CHECK_VALUE(lu.K == H && lu.N == I && ld.K == I && ld.N == H, "gate / up must be H -> I and down I -> H");
    TORCH_CHECK_VALUE(lu.device == lg.device && ld.device == lg.device, "the three layers must be on one device");
    const at::Tensor x2 = flat_half(x, H, lg.device, "x");
    const int64_t M = x2.size(0);
    TORCH_CHECK_VALUE(M >= 1 && M <= 16, "mlp_decode handles 1..16 rows, got ", M);
    at::Tensor y = at::empty(out_sizes(out_shape, M, H), x2.options());
    at::Tensor go, uo;
    if (intermediates) {
        go = at::empty({M, (int64_t)I}, x2.options());
        uo = at::empty({M, (int64_t)I}, x2.options());
    }
    Launch L(lg.device);
    const size_t need = q4_mlp_decode_workspace_bytes((int)M, H, I);
    at::Tensor ws;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        at::Tensor& slot = g_mlp_buffers[MlpKey{lg.device.index(), L.stream, (int)M, H, I}];
        if (!slot.defined()) slot = at::zeros({(int64_t)need}, at::TensorOptions().dtype(at::kByte).device(lg.device));
        ws = slot;
    }
    const q4_layer_t dg{lg.qweight, lg.qzeros, lg.scales}, du{lu.qweight, lu.qzeros, lu.scales}, dd{ld.qweight, ld.qzeros, ld.scales};
    const int rc = q4_mlp_decode_f16(x2.data_ptr(), &dg, &du, &dd, (int)groupsize, intermediates ? go.data_ptr() : nullptr,
                                     intermediates ? uo.data_ptr() : nullptr, y.data_ptr(), (int)M, H, I, ws.data_ptr(),
                                     (size_t)ws.numel(), L.stream);
    if (rc != Q4_OK) {
        if (rc == Q4_ERR_LAUNCH) ws.zero_();
        raise_q4(rc, "q4_mlp_decode_f16");
    }
    if (intermediates) return {y, go, uo};
    return {y};
}

// 1 when a wait inside some fused MLP launch on this device hit its poll limit (synchronises; for tests).
bool mlp_decode_gave_up() {
    std::vector<std::pair<at::Tensor, size_t>> all;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        for (auto& kv : g_mlp_buffers)
            all.emplace_back(kv.second, q4_mlp_decode_status_offset(kv.first.M, kv.first.H, kv.first.I));
    }
    for (auto& p : all)
        if (p.first.narrow(0, (int64_t)p.second, 4).any().item<bool>()) return true;
    return false;
}

struct LoraPair {
    const void* la = nullptr;
    const void* lb = nullptr;
    int R = 0, sr = 0, sc = 0, f32 = 0;
};
// la: [rows, R] fp16 contiguous; lb: [R, cols] fp16 / fp32 view with positive strides
LoraPair check_lora(const c10::optional<at::Tensor>& la, const c10::optional<at::Tensor>& lb, int64_t rows, int64_t cols,
                    const c10::Device& dev) {
    LoraPair p;
    if (!la.has_value() && !lb.has_value()) return p;
    TORCH_CHECK_VALUE(la.has_value() && lb.has_value(), "both LoRA operands are required");
    const at::Tensor& a = *la;
    const at::Tensor& b = *lb;
    TORCH_CHECK_VALUE(a.scalar_type() == at::kHalf, "the rank-R activation operand must be float16");
    TORCH_CHECK_VALUE(b.scalar_type() == at::kHalf || b.scalar_type() == at::kFloat, "the adapter matrix must be float16 or float32");
    const int64_t R = a.size(-1);
    TORCH_CHECK_VALUE(a.dim() == 2 && a.size(0) == rows && b.dim() == 2 && b.size(0) == R && b.size(1) == cols,
                      "LoRA operand shapes do not match");
    TORCH_CHECK_VALUE(R % 8 == 0 && R >= 8 && R <= 64, "LoRA rank must be a multiple of 8 in [8, 64] for the fused path");
    TORCH_CHECK_VALUE(a.is_contiguous() && a.device() == dev && b.device() == dev, "LoRA operands must be on the same device");
    TORCH_CHECK_VALUE(b.stride(0) >= 1 && b.stride(1) >= 1, "the adapter matrix must have positive strides");
    p.la = a.data_ptr(); p.lb = b.data_ptr(); p.R = (int)R; p.sr = (int)b.stride(0); p.sc = (int)b.stride(1);
    p.f32 = b.scalar_type() == at::kFloat;
    return p;
}

// out[m, p] = in[m, idx[p]]: activations gathered through the row sort of an act-order layer's weights (or grad_input
// gathered back through the inverse permutation).  `idx` int32 [K] on the same device.
at::Tensor permute_cols(const at::Tensor& in2, const at::Tensor& idx, void* stream) {
    const int64_t M = in2.size(0), K = in2.size(1);
    TORCH_CHECK_VALUE(idx.scalar_type() == at::kInt && idx.dim() == 1 && idx.size(0) == K && idx.is_contiguous() &&
                      idx.device() == in2.device(), "the column index must be a contiguous int32 [K] tensor on the same device");
    at::Tensor out = at::empty_like(in2);
    const int rc = q4_permute_cols_f16(in2.data_ptr(), idx.data_ptr<int32_t>(), out.data_ptr(), (int)M, (int)K, stream);
    if (rc != Q4_OK) raise_q4(rc, "q4_permute_cols_f16");
    return out;
}

at::Tensor gemm_fwd(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& qzeros, const at::Tensor& scales,
                    const c10::optional<at::Tensor>& g_idx, int64_t groupsize, const c10::optional<at::Tensor>& bias,
                    const c10::optional<at::Tensor>& xa, const c10::optional<at::Tensor>& lora_bt, double lora_scale,
                    const c10::optional<std::vector<int64_t>>& out_shape, const c10::optional<at::Tensor>& in_perm) {
    const Layer l = check_layer(qweight, qzeros, scales, g_idx, groupsize);
    at::Tensor x2 = flat_half(x, l.K, l.device, "x");
    const int64_t M = x2.size(0);
    if (M == 0) return at::empty(out_sizes(out_shape, 0, l.N), x2.options());
    const void* bp = nullptr;
    if (bias.has_value()) {
        TORCH_CHECK_VALUE(bias->scalar_type() == at::kHalf && bias->dim() == 1 && bias->size(0) == l.N && bias->is_contiguous() &&
                          bias->device() == l.device, "bias must be a contiguous float16 [N] tensor on the same device");
        bp = bias->data_ptr();
    }
    const LoraPair lp = check_lora(xa, lora_bt, M, l.N, l.device);
    at::Tensor o = at::empty(out_sizes(out_shape, M, l.N), x2.options());
    Launch L(l.device);
    if (in_perm.has_value()) x2 = permute_cols(x2, *in_perm, L.stream);     // `qweight` holds the rows in that order
    size_t have = 0;
    void* ws = scratch_workspace(l.device, L.stream, q4_gemm_workspace_bytes(1, (int)M, l.K, l.N), &have);
    const int rc = q4_gemm_fwd_f16(x2.data_ptr(), l.qweight, l.qzeros, l.scales, l.g_idx, l.groupsize, bp, lp.la, lp.lb, lp.sr,
                                   lp.sc, lp.f32, (float)lora_scale, lp.R, o.data_ptr(), (int)M, l.K, l.N, l.G, ws, have, L.stream);
    if (rc != Q4_OK) raise_q4(rc, "q4_gemm_fwd_f16");
    return o;
}

at::Tensor gemm_bwd_dx(const at::Tensor& dy, const at::Tensor& qweight, const at::Tensor& qzeros, const at::Tensor& scales,
                       const c10::optional<at::Tensor>& g_idx, int64_t groupsize, const c10::optional<at::Tensor>& dyb,
                       const c10::optional<at::Tensor>& lora_a, double lora_scale,
                       const c10::optional<std::vector<int64_t>>& out_shape,
                       const c10::optional<std::pair<int64_t, double>>& dropout, const c10::optional<at::Tensor>& out_perm) {
    const Layer l = check_layer(qweight, qzeros, scales, g_idx, groupsize);
    const at::Tensor dy2 = flat_half(dy, l.N, l.device, "grad_output");
    const int64_t M = dy2.size(0);
    if (M == 0) return at::empty(out_sizes(out_shape, 0, l.K), dy2.options());
    const LoraPair lp = check_lora(dyb, lora_a, M, l.K, l.device);
    at::Tensor o = at::empty(out_sizes(out_shape, M, l.K), dy2.options());
    q4_dropout_t d;
    const bool has_drop = fill_drop(dropout, &d);
    Launch L(l.device);
    size_t have = 0;
    void* ws = scratch_workspace(l.device, L.stream, q4_gemm_workspace_bytes(0, (int)M, l.K, l.N), &have);
    const int rc = q4_gemm_bwd_dx_f16(dy2.data_ptr(), l.qweight, l.qzeros, l.scales, l.g_idx, l.groupsize, lp.la, lp.lb, lp.sr,
                                      lp.sc, lp.f32, (float)lora_scale, lp.R, o.data_ptr(), (int)M, l.K, l.N, l.G,
                                      has_drop ? &d : nullptr, ws, have, L.stream);
    if (rc != Q4_OK) raise_q4(rc, "q4_gemm_bwd_dx_f16");
    if (out_perm.has_value())               // the rows of `qweight` are sorted: grad_input back into the original order
        return permute_cols(o.view({M, (int64_t)l.K}), *out_perm, L.stream).view(o.sizes());
    return o;
}

// One layer of a grouped GEMM: (qweight, qzeros, scales, bias | None, rank-R operand | None, adapter matrix view | None,
// adapter scale, dropout (seed, p) | None).  Forward: bias, xa, lora_B^T view; grad-input: no bias, dyb, lora_A.
using GroupLayer = std::tuple<at::Tensor, at::Tensor, at::Tensor, c10::optional<at::Tensor>, c10::optional<at::Tensor>,
                              c10::optional<at::Tensor>, double, c10::optional<std::pair<int64_t, double>>>;

// y_i = x @ W_i (+ bias_i) (+ scale_i * xa_i @ lora_bt_i) for 2..4 layers in one launch; raises when the shape does not
// qualify (the caller falls back to per-layer calls).
std::vector<at::Tensor> gemm_grouped_fwd(const at::Tensor& x, const std::vector<GroupLayer>& layers, int64_t groupsize) {
    const size_t n = layers.size();
    TORCH_CHECK_VALUE(n >= 2 && n <= 4, "gemm_grouped_fwd takes 2..4 layers");
    q4_gemm_layer_t desc[4];
    std::vector<at::Tensor> outs;
    at::Tensor x2;
    int64_t M = 0, K = 0;
    c10::optional<c10::Device> dev;
    for (size_t i = 0; i < n; ++i) {
        const Layer l = check_layer(std::get<0>(layers[i]), std::get<1>(layers[i]), std::get<2>(layers[i]), c10::nullopt, groupsize);
        if (i == 0) { dev = l.device; K = l.K; x2 = flat_half(x, K, *dev, "x"); M = x2.size(0); }
        TORCH_CHECK_VALUE(l.device == *dev && l.K == K, "grouped layers must share the device and K");
        const auto& bias = std::get<3>(layers[i]);
        const void* bp = nullptr;
        if (bias.has_value()) {
            TORCH_CHECK_VALUE(bias->scalar_type() == at::kHalf && bias->dim() == 1 && bias->size(0) == l.N && bias->is_contiguous() &&
                              bias->device() == *dev, "bias must be a contiguous float16 [N] tensor on the same device");
            bp = bias->data_ptr();
        }
        const LoraPair lp = check_lora(std::get<4>(layers[i]), std::get<5>(layers[i]), M, l.N, *dev);
        at::Tensor o = at::empty({M, (int64_t)l.N}, x2.options());
        desc[i] = q4_gemm_layer_t{x2.data_ptr(), l.qweight, l.qzeros, l.scales, bp, lp.la, lp.lb, lp.sr, lp.sc, lp.f32,
                                  (float)std::get<6>(layers[i]), lp.R, o.data_ptr(), l.N, nullptr};
        outs.push_back(o);
    }
    Launch L(*dev);
    const int rc = q4_gemm_grouped_fwd_f16(desc, (int)n, (int)groupsize, (int)M, (int)K, L.stream);
    if (rc != Q4_OK) raise_q4(rc, "q4_gemm_grouped_fwd_f16");
    return outs;
}

// dx = sum_i ( dy_i @ W_i^T + mask_i * scale_i * dyb_i @ lora_a_i ) in one launch and one ordered reduction.
at::Tensor gemm_grouped_bwd_dx(const std::vector<at::Tensor>& dys, const std::vector<GroupLayer>& layers, int64_t groupsize,
                               const c10::optional<std::vector<int64_t>>& out_shape) {
    const size_t n = layers.size();
    TORCH_CHECK_VALUE(n >= 2 && n <= 4 && dys.size() == n, "gemm_grouped_bwd_dx takes 2..4 layers and one grad_output per layer");
    q4_gemm_layer_t desc[4];
    q4_dropout_t drops[4];
    std::vector<at::Tensor> keep;
    int n32[4];
    int64_t M = 0, K = 0;
    c10::optional<c10::Device> dev;
    for (size_t i = 0; i < n; ++i) {
        const Layer l = check_layer(std::get<0>(layers[i]), std::get<1>(layers[i]), std::get<2>(layers[i]), c10::nullopt, groupsize);
        if (i == 0) { dev = l.device; K = l.K; }
        TORCH_CHECK_VALUE(l.device == *dev && l.K == K, "grouped layers must share the device and K");
        at::Tensor dy2 = flat_half(dys[i], l.N, *dev, "grad_output");
        if (i == 0) M = dy2.size(0);
        TORCH_CHECK_VALUE(dy2.size(0) == M, "grouped layers must share the number of rows");
        keep.push_back(dy2);
        const LoraPair lp = check_lora(std::get<4>(layers[i]), std::get<5>(layers[i]), M, K, *dev);
        const bool has_drop = fill_drop(std::get<7>(layers[i]), &drops[i]);
        desc[i] = q4_gemm_layer_t{dy2.data_ptr(), l.qweight, l.qzeros, l.scales, nullptr, lp.la, lp.lb, lp.sr, lp.sc, lp.f32,
                                  (float)std::get<6>(layers[i]), lp.R, nullptr, l.N, has_drop ? &drops[i] : nullptr};
        n32[i] = l.N;
    }
    at::Tensor dx = at::empty(out_sizes(out_shape, M, K), keep[0].options());
    Launch L(*dev);
    size_t have = 0;
    void* ws = scratch_workspace(*dev, L.stream, q4_gemm_grouped_workspace_bytes(0, (int)n, (int)M, (int)K, n32), &have);
    const int rc = q4_gemm_grouped_bwd_dx_f16(desc, (int)n, (int)groupsize, dx.data_ptr(), (int)M, (int)K, ws, have, L.stream);
    if (rc != Q4_OK) raise_q4(rc, "q4_gemm_grouped_bwd_dx_f16");
    return dx;
}

at::Tensor lora_down(const at::Tensor& inp, const at::Tensor& w, const c10::optional<std::pair<int64_t, double>>& dropout) {
    TORCH_CHECK_VALUE(inp.is_cuda() && inp.scalar_type() == at::kHalf && inp.dim() == 2 && inp.is_contiguous(),
                      "inp must be a contiguous float16 [M, C] CUDA tensor");
    const int64_t M = inp.size(0), C = inp.size(1);
    TORCH_CHECK_VALUE(w.dim() == 2 && w.size(1) == C && w.device() == inp.device(), "w must be an [R, C] view on the same device");
    TORCH_CHECK_VALUE(w.scalar_type() == at::kHalf || w.scalar_type() == at::kFloat, "w must be float16 or float32");
    const int64_t R = w.size(0);
    at::Tensor o = at::empty({M, R}, inp.options());
    if (M == 0) return o;
    TORCH_CHECK_VALUE(R >= 1 && R <= 64 && C % 32 == 0, "lora_down needs 1 <= R <= 64 and C % 32 == 0");
    TORCH_CHECK_VALUE(w.stride(0) >= 1 && w.stride(1) >= 1, "w must have positive strides");
    q4_dropout_t d;
    const bool has_drop = fill_drop(dropout, &d);
    Launch L(inp.device());
    const int rc = q4_lora_down_f16(inp.data_ptr(), w.data_ptr(), (int)w.stride(0), (int)w.stride(1), w.scalar_type() == at::kFloat,
                                    o.data_ptr(), (int)M, (int)C, (int)R, has_drop ? &d : nullptr, L.stream);
    if (rc != Q4_OK) raise_q4(rc, "q4_lora_down_f16");
    return o;
}

std::pair<at::Tensor, at::Tensor> lora_grad_pair(const at::Tensor& p1, const at::Tensor& in1, const at::Tensor& p2,
                                                 const at::Tensor& in2, double alpha,
                                                 const c10::optional<std::pair<int64_t, double>>& dropout) {
    for (const auto& pr : {std::make_pair(&p1, &in1), std::make_pair(&p2, &in2)}) {
        const at::Tensor& p = *pr.first;
        const at::Tensor& in = *pr.second;
        TORCH_CHECK_VALUE(p.is_cuda() && p.scalar_type() == at::kHalf && p.dim() == 2 && p.is_contiguous(),
                          "p must be a contiguous float16 [M, R] CUDA tensor");
        TORCH_CHECK_VALUE(in.scalar_type() == at::kHalf && in.dim() == 2 && in.is_contiguous() && in.device() == p.device() &&
                          in.size(0) == p.size(0), "inp must be a contiguous float16 [M, C] tensor on the same device");
    }
    TORCH_CHECK_VALUE(p1.sizes() == p2.sizes() && p1.device() == p2.device(), "the two rank-R operands must share shape and device");
    const int64_t M = p1.size(0), R = p1.size(1), C1 = in1.size(1), C2 = in2.size(1);
    TORCH_CHECK_VALUE(R >= 2 && R <= 32 && R % 2 == 0 && C1 % 8 == 0 && C2 % 8 == 0, "lora_grad needs an even R in 2..32 and C % 8 == 0");
    const auto opt = at::TensorOptions().dtype(at::kFloat).device(p1.device());
    if (M == 0) return {at::zeros({R, C1}, opt), at::zeros({C2, R}, opt)};
    at::Tensor o1 = at::empty({R, C1}, opt), o2 = at::empty({C2, R}, opt);
    q4_dropout_t d;
    const bool has_drop = fill_drop(dropout, &d);
    Launch L(p1.device());
    size_t have = 0;
    const size_t need = q4_lora_grad_workspace_bytes((int)M, (int)C1, (int)R) + q4_lora_grad_workspace_bytes((int)M, (int)C2, (int)R);
    void* ws = scratch_workspace(p1.device(), L.stream, need, &have);
    const int rc = q4_lora_grad_pair_f32(p1.data_ptr(), in1.data_ptr(), o1.data_ptr<float>(), (int)C1, 1, (int)C1,
                                         p2.data_ptr(), in2.data_ptr(), o2.data_ptr<float>(), 1, (int)R, (int)C2,
                                         (float)alpha, (int)M, (int)R, has_drop ? &d : nullptr, ws, have, L.stream);
    if (rc != Q4_OK) raise_q4(rc, "q4_lora_grad_pair_f32");
    return {o1, o2};
}

// Clears the cached GEMV accumulators of every stream (after an aborted run, or when a caller is unsure).
void reset_workspaces() {
    std::lock_guard<std::mutex> lock(g_mutex);
    for (auto& kv : g_buffers)
        if (kv.second.zeroed.defined()) kv.second.zeroed.zero_();
    for (auto& kv : g_mlp_buffers) kv.second.zero_();          // all zero = the state before a workspace's first use
}

// True when the cached GEMV accumulators of every stream are all zero (synchronises; for tests and debugging).
bool workspaces_are_zero() {
    std::lock_guard<std::mutex> lock(g_mutex);
    for (auto& kv : g_buffers)
        if (kv.second.zeroed.defined() && kv.second.zeroed.any().item<bool>()) return false;
    return true;
}

void drop_workspaces() {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_buffers.clear();
    g_mlp_buffers.clear();
    g_retired.clear();
}

}  // namespace

PYBIND11_MODULE(_q4_host, m) {
    m.doc() = "compiled host binding of libq4gptq (checks, current stream, workspaces, launch)";
    m.def("set_error_class", [](py::object cls) { g_error_class = std::move(cls); });
    // File-scope objects would be destroyed when the library is unloaded, after the interpreter and the HIP runtime
    // have shut down: release what they hold while both are still alive.
    py::module_::import("atexit").attr("register")(py::cpp_function([] {
        g_error_class = py::object();
        drop_workspaces();
    }));
    m.def("abi_version", [] { return q4_abi_version(); });
    m.def("dequant", &dequant, py::arg("qweight"), py::arg("qzeros"), py::arg("scales"), py::arg("g_idx"), py::arg("groupsize"),
          py::arg("out") = py::none());
    m.def("gemv", &gemv, py::arg("x"), py::arg("qweight"), py::arg("qzeros"), py::arg("scales"), py::arg("g_idx"),
          py::arg("groupsize"), py::arg("out") = py::none(), py::arg("accumulate") = false, py::arg("out_shape") = py::none());
    m.def("gemv_grouped", &gemv_grouped, py::arg("xs"), py::arg("layers"), py::arg("groupsize"), py::arg("outs") = py::none(),
          py::arg("accumulate") = false);
    m.def("gemm_fwd", &gemm_fwd, py::arg("x"), py::arg("qweight"), py::arg("qzeros"), py::arg("scales"), py::arg("g_idx"),
          py::arg("groupsize"), py::arg("bias") = py::none(), py::arg("xa") = py::none(), py::arg("lora_bt") = py::none(),
          py::arg("lora_scale") = 1.0, py::arg("out_shape") = py::none(), py::arg("in_perm") = py::none());
    m.def("gemm_bwd_dx", &gemm_bwd_dx, py::arg("dy"), py::arg("qweight"), py::arg("qzeros"), py::arg("scales"), py::arg("g_idx"),
          py::arg("groupsize"), py::arg("dyb") = py::none(), py::arg("lora_a") = py::none(), py::arg("lora_scale") = 1.0,
          py::arg("out_shape") = py::none(), py::arg("dropout") = py::none(), py::arg("out_perm") = py::none());
    m.def("gemm_grouped_fwd", &gemm_grouped_fwd, py::arg("x"), py::arg("layers"), py::arg("groupsize"));
    m.def("gemm_grouped_bwd_dx", &gemm_grouped_bwd_dx, py::arg("dys"), py::arg("layers"), py::arg("groupsize"),
          py::arg("out_shape") = py::none());
    m.def("lora_down", &lora_down, py::arg("inp"), py::arg("w"), py::arg("dropout") = py::none());
    m.def("lora_grad_pair", &lora_grad_pair, py::arg("p1"), py::arg("inp1"), py::arg("p2"), py::arg("inp2"), py::arg("alpha"),
          py::arg("dropout") = py::none());
    m.def("mlp_decode", &mlp_decode, py::arg("x"), py::arg("gate"), py::arg("up"), py::arg("down"), py::arg("groupsize"),
          py::arg("intermediates") = false, py::arg("out_shape") = py::none());
    m.def("mlp_decode_gave_up", &mlp_decode_gave_up);
    m.def("reset_workspaces", &reset_workspaces);
    m.def("workspaces_are_zero", &workspaces_are_zero);
    m.def("drop_workspaces", &drop_workspaces);
}
