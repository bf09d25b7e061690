// Host side of the attention path above the C ABI, in C++ (the reference's host side is Rust, for
// which this environment has no toolchain).  It mirrors the reference's operator interface for this
// path -- same names, argument meaning and error behaviour -- so that a Rust shim is a line-by-line
// transliteration:
//
//   flame::sdpa::forward / forward_train            src/sdpa.rs:85-207
//   flame::attention::sdpa / attend / attention_impl / build_causal_mask
//                                                   src/attention/sdpa.rs:521-558, :395-458, :11-34
//   flame::autograd::{AutogradContext, Op::FlashAttention node, flash_attention_backward}
//                                                   src/autograd.rs:289-296, :672-795, :3824-3916
//   flame::autograd_v4::{SdpaConfig, SdpaSave, SdpaCtx, sdpa_forward, sdpa_backward}
//                                                   src/autograd_v4/ops/sdpa.rs:21-96, :98-326, :826-1009
//   flame::SageAttention                            src/sage_attention.rs:21-171
//   flame::autograd_v4::{SdpaStats, SdpaHooks, register_sdpa_hooks}
//                                                   src/autograd_v4/ops/sdpa.rs:56-79, :1063-1074
//   flame::perf_telemetry::{telemetry_enabled, log_sdpa_event}
//                                                   src/perf_telemetry.rs:7-40, :60-150
//
// Only what the path needs of the tensor type is here: a reference-counted device buffer with a
// shape, element strides, an offset and a dtype (the reference's Tensor supplies exactly these to
// the FFI: src/tensor.rs:558, :2637, :2657).  Header-only; link against libflame_attn_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <chrono>
#include <functional>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <tuple>
#include <unordered_map>
#include <utility>
#include <vector>

#include "../../include/flame_attn.h"

namespace flame {

// ------------------------------------------------------------------------------------ errors
// The reference's `Error` enum, reduced to the variants this path raises (src/error.rs).
struct Error {
    enum Kind { InvalidInput, Unsupported, Cuda, InvalidOperation, OutOfMemory } kind;
    std::string message;
};

template <class T>
class Result {
   public:
    Result(T v) : value_(std::move(v)) {}
    Result(Error e) : error_(std::move(e)) {}
    bool ok() const { return value_.has_value(); }
    const T& value() const { return *value_; }
    T& value() { return *value_; }
    const Error& error() const { return *error_; }

   private:
    std::optional<T> value_;
    std::optional<Error> error_;
};

inline Error invalid(std::string m) { return Error{Error::InvalidInput, std::move(m)}; }
inline Error unsupported(std::string m) { return Error{Error::Unsupported, std::move(m)}; }
inline Error cuda_error(const std::string& what, int code) {
    return Error{Error::Cuda, what + " HIP error: " + std::to_string(code)};   // src/sdpa.rs:680-682
}

// ------------------------------------------------------------------------------------ tensor
enum class DType { BF16, F32, U8, I8, I32 };
inline size_t dtype_size(DType d) { return d == DType::BF16 ? 2 : (d == DType::U8 || d == DType::I8) ? 1 : 4; }

class Tensor {
   public:
    Tensor() = default;

    static Result<Tensor> empty(std::vector<int64_t> shape, DType dtype) {
        int64_t n = 1;
        for (auto d : shape) {
            if (d <= 0) return invalid("empty: non-positive dimension");
            n *= d;
        }
        void* p = nullptr;
        hipError_t e = hipMalloc(&p, (size_t)n * dtype_size(dtype));
        if (e != hipSuccess) return cuda_error("hipMalloc", (int)e);
        Tensor t;
        t.storage_ = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
        t.shape_ = std::move(shape);
        t.strides_ = contiguous_strides(t.shape_);
        t.dtype_ = dtype;
        return t;
    }
    static Result<Tensor> from_host(const void* src, std::vector<int64_t> shape, DType dtype) {
        auto r = empty(std::move(shape), dtype);
        if (!r.ok()) return r;
        hipError_t e = hipMemcpy(r.value().data(), src, (size_t)r.value().numel() * dtype_size(dtype), hipMemcpyHostToDevice);
        if (e != hipSuccess) return cuda_error("hipMemcpy", (int)e);
        return r;
    }
    // contiguous tensors only
    Result<bool> to_host(void* dst) const {
        if (!is_contiguous()) return unsupported("to_host: tensor is a strided view");
        hipError_t e = hipMemcpy(dst, data(), (size_t)numel() * dtype_size(dtype_), hipMemcpyDeviceToHost);
        if (e != hipSuccess) return cuda_error("hipMemcpy", (int)e);
        return true;
    }

    const std::vector<int64_t>& shape() const { return shape_; }
    const std::vector<int64_t>& strides() const { return strides_; }
    int64_t offset() const { return offset_; }
    DType dtype() const { return dtype_; }
    int64_t numel() const {
        int64_t n = 1;
        for (auto d : shape_) n *= d;
        return n;
    }
    void* base() const { return storage_.get(); }
    void* data() const { return static_cast<char*>(storage_.get()) + offset_ * (int64_t)dtype_size(dtype_); }
    bool defined() const { return storage_ != nullptr; }
    uint64_t id() const { return (uint64_t)(uintptr_t)storage_.get() ^ ((uint64_t)offset_ << 1); }
    bool requires_grad = false;

    bool is_contiguous() const { return strides_ == contiguous_strides(shape_); }
    // view with permuted dimensions (no copy), e.g. [B,N,H,D] -> [B,H,N,D] with {0,2,1,3}
    Tensor permute(const std::vector<int>& order) const {
        Tensor t = *this;
        for (size_t i = 0; i < order.size(); ++i) {
            t.shape_[i] = shape_[order[i]];
            t.strides_[i] = strides_[order[i]];
        }
        return t;
    }
    // view of the first n elements of the last dimension (no copy)
    Tensor narrow_last(int64_t n) const {
        Tensor t = *this;
        t.shape_.back() = n;
        return t;
    }
    Tensor reshape_contiguous(std::vector<int64_t> shape) const {
        Tensor t = *this;
        t.shape_ = std::move(shape);
        t.strides_ = contiguous_strides(t.shape_);
        return t;
    }

    static std::vector<int64_t> contiguous_strides(const std::vector<int64_t>& shape) {
        std::vector<int64_t> st(shape.size(), 1);
        for (int i = (int)shape.size() - 2; i >= 0; --i) st[i] = st[i + 1] * shape[i + 1];
        return st;
    }

   private:
    std::shared_ptr<void> storage_;
    std::vector<int64_t> shape_, strides_;
    int64_t offset_ = 0;
    DType dtype_ = DType::BF16;
};

namespace detail {

// trap_is_bf16 of the reference (src/tensor/contracts.rs:22-33): non-bf16 -> InvalidInput
inline std::optional<Error> trap_is_bf16(const char* what, const Tensor& t) {
    if (t.dtype() != DType::BF16) return invalid(std::string(what) + ": expected BF16 tensor");
    return std::nullopt;
}

struct Dims {
    int B, H, Sq, Sk, D;
};

// shape / mask validation of forward_inner (src/sdpa.rs:330-374), same messages' meaning
inline Result<Dims> validate(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask) {
    for (const Tensor* t : {&q, &k, &v})
        if (t->shape().size() != 4) return invalid("expected 4D tensor [B,H,S,D]");
    const auto &qs = q.shape(), &ks = k.shape(), &vs = v.shape();
    if (!(qs[0] == ks[0] && qs[0] == vs[0] && qs[1] == ks[1] && qs[1] == vs[1])) return invalid("batch/head mismatch");
    if (!(qs[3] == ks[3] && qs[3] == vs[3])) return invalid("embed mismatch");
    if (ks[2] != vs[2]) return invalid("sequence mismatch: k_len != v_len");
    if (mask) {
        const auto& ms = mask->shape();
        if (ms.size() != 4) return invalid("mask must be 4D [B,H,Q,K]");
        if (!(ms[0] == qs[0] || ms[0] == 1) || !(ms[1] == qs[1] || ms[1] == 1) || ms[2] != qs[2] || ms[3] != ks[2])
            return invalid("mask dims not broadcastable to [B,H,Q,K]");
    }
    if (auto e = trap_is_bf16("sdpa.forward q", q)) return *e;
    if (auto e = trap_is_bf16("sdpa.forward k", k)) return *e;
    if (auto e = trap_is_bf16("sdpa.forward v", v)) return *e;
    return Dims{(int)qs[0], (int)qs[1], (int)qs[2], (int)ks[2], (int)qs[3]};
}

inline bool abi_friendly(const Tensor& t) {
    const auto& st = t.strides();
    return st[3] == 1 && ((st[0] | st[1] | st[2] | t.offset()) & 7) == 0;
}

// binary keep-mask of any supported dtype -> contiguous uint8 keep-mask + broadcast strides
inline Result<std::pair<Tensor, std::vector<int64_t>>> prepare_mask(const Tensor& mask, const Dims& d) {
    Tensor m8 = mask;
    if (mask.dtype() != DType::U8) {
        if (!mask.is_contiguous()) return unsupported("non-contiguous non-uint8 mask");
        if (mask.dtype() != DType::BF16 && mask.dtype() != DType::F32) return invalid("mask dtype must be U8, BF16 or F32");
        auto r = Tensor::empty(mask.shape(), DType::U8);
        if (!r.ok()) return r.error();
        const int rc = flame_attn_convert_keep_mask(mask.data(), mask.dtype() == DType::BF16 ? FLAME_ATTN_DTYPE_BF16 : FLAME_ATTN_DTYPE_F32,
                                                    r.value().data(), mask.numel(), nullptr);
        if (rc != 0) return cuda_error("flame_attn_convert_keep_mask", rc);
        m8 = r.value();
    }
    std::vector<int64_t> st(4);
    const int64_t full[4] = {d.B, d.H, d.Sq, d.Sk};
    for (int i = 0; i < 4; ++i) st[i] = (m8.shape()[i] == 1 && full[i] != 1) ? 0 : m8.strides()[i];
    return std::make_pair(m8, st);
}

struct FwdOut {
    Tensor o, stats;
};

inline Result<FwdOut> run_forward(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask, bool causal,
                                  std::optional<float> scale, bool want_stats, float dropout_p = 0.f, uint64_t dropout_seed = 0,
                                  int draw_chunk_q = 0, int draw_chunk_kv = 0) {
    auto dv = validate(q, k, v, mask);
    if (!dv.ok()) return dv.error();
    const Dims d = dv.value();
    for (const Tensor* t : {&q, &k, &v})
        if (t->strides()[3] != 1 || (d.D % 8 == 0 && !abi_friendly(*t)))
            return unsupported("tensor view needs D stride 1 and 16-byte aligned rows; make it contiguous first");
    auto o = Tensor::empty({d.B, d.H, d.Sq, d.D}, DType::BF16);      // O = q.shape, contiguous (src/sdpa.rs:631)
    if (!o.ok()) return o.error();
    Tensor stats;
    if (want_stats) {
        auto s = Tensor::empty({(int64_t)d.B * d.H, d.Sq}, DType::F32);   // [B*H, Sq] fp32 (src/sdpa.rs:712-722)
        if (!s.ok()) return s.error();
        stats = s.value();
    }
    Tensor m8;
    std::vector<int64_t> mst;
    if (mask) {
        auto pm = prepare_mask(*mask, d);
        if (!pm.ok()) return pm.error();
        m8 = pm.value().first;
        mst = pm.value().second;
    }
    const float sc = scale.value_or(1.0f / std::sqrt((float)d.D));
    int rc;
    if (dropout_p != 0.f) {
        rc = flame_attn_fwd_dropout_tiled_bf16(
            q.base(), k.base(), v.base(), o.value().base(), want_stats ? stats.base() : nullptr, d.B, d.H, d.Sq, d.Sk, d.D, sc,
            q.strides().data(), k.strides().data(), v.strides().data(), o.value().strides().data(), q.offset(), k.offset(),
            v.offset(), 0, 0, causal ? 1 : 0, nullptr, mask ? static_cast<const uint8_t*>(m8.data()) : nullptr,
            mask ? mst.data() : nullptr, dropout_p, dropout_seed, draw_chunk_q, draw_chunk_kv, nullptr);
        if (rc != 0 && rc != FLAME_ATTN_ERR_UNSUPPORTED) return cuda_error("flame_attn_fwd_dropout_tiled_bf16", rc);
    } else {
        rc = flame_attn_fwd_bf16(q.base(), k.base(), v.base(), o.value().base(), want_stats ? stats.base() : nullptr,
                                 d.B, d.H, d.Sq, d.Sk, d.D, sc, q.strides().data(), k.strides().data(),
                                 v.strides().data(), o.value().strides().data(), q.offset(), k.offset(), v.offset(), 0, 0,
                                 causal ? 1 : 0, nullptr, mask ? static_cast<const uint8_t*>(m8.data()) : nullptr,
                                 mask ? mst.data() : nullptr, nullptr /* default stream, as the reference */);
    }
    if (rc == FLAME_ATTN_ERR_UNSUPPORTED) {
        // forward_bf16's last branch (src/sdpa.rs:543-587 -> forward_bf16_fallback, :788-961): whatever the fused
        // kernels do not serve (a head dim that is not a multiple of 8 or lies above 512, a mask above 128) goes
        // through materialised scores, one band of query rows at a time
        const size_t wsb = flame_attn_materialised_workspace_bytes(d.B, d.H, d.Sq, d.Sk, d.D, d.D, 0);
        auto ws = Tensor::empty({(int64_t)wsb}, DType::U8);
        if (!ws.ok()) return ws.error();
        const int rm = flame_attn_fwd_materialised_bf16(
            q.base(), k.base(), v.base(), o.value().base(), want_stats ? stats.base() : nullptr, d.B, d.H, d.Sq, d.Sk, d.D, d.D, sc,
            q.strides().data(), k.strides().data(), v.strides().data(), o.value().strides().data(), q.offset(), k.offset(), v.offset(),
            0, 0, causal ? 1 : 0, nullptr, mask ? static_cast<const uint8_t*>(m8.data()) : nullptr, mask ? mst.data() : nullptr, nullptr,
            FLAME_ATTN_DTYPE_F32, nullptr, dropout_p, dropout_seed, draw_chunk_q, draw_chunk_kv, ws.value().data(), wsb, nullptr);
        if (rm == FLAME_ATTN_ERR_UNSUPPORTED) return unsupported("flame_attn_fwd_materialised_bf16: layout not served (or rocBLAS missing)");
        if (rm != 0) return cuda_error("flame_attn_fwd_materialised_bf16", rm);
        return FwdOut{o.value(), stats};
    }
    if (rc != 0) return cuda_error("flame_attn_fwd_bf16", rc);
    return FwdOut{o.value(), stats};
}

}  // namespace detail

// ------------------------------------------------------------------------------------ autograd (default engine)
namespace autograd {

// Op::FlashAttention and its saved set {Q, K, V, O, Stats(, mask)} (src/autograd.rs:289-296, src/sdpa.rs:170-201)
struct FlashAttentionNode {
    uint64_t output_id = 0;
    Tensor query, key, value, output, stats;
    std::optional<Tensor> mask;
    float scale = 0.f;
    bool causal = false;
    float dropout_p = 0.f;            // set by the v4 operator only (autograd_v4::SdpaCtx)
    uint64_t dropout_seed = 0;
    int draw_chunk_q = 0, draw_chunk_kv = 0;    // tiles of a chunked draw, 0 = the whole axis
};

class AutogradContext {
   public:
    static bool is_recording() { return state().recording; }
    static void set_recording(bool on) { state().recording = on; }
    static void record_op(FlashAttentionNode node) {
        std::lock_guard<std::mutex> g(state().mu);
        state().tape.push_back(std::move(node));
    }
    static std::optional<FlashAttentionNode> find(const Tensor& output) {
        std::lock_guard<std::mutex> g(state().mu);
        for (auto it = state().tape.rbegin(); it != state().tape.rend(); ++it)
            if (it->output_id == output.id()) return *it;
        return std::nullopt;
    }
    static void clear() {
        std::lock_guard<std::mutex> g(state().mu);
        state().tape.clear();
    }
    // bytes this node keeps alive between forward and backward that a materialised softmax would not
    static size_t saved_activation_bytes(const FlashAttentionNode& n) {
        return (size_t)n.output.numel() * 2 + (size_t)n.stats.numel() * 4;
    }

   private:
    struct State {
        bool recording = false;
        std::mutex mu;
        std::vector<FlashAttentionNode> tape;
    };
    static State& state() {
        static State s;
        return s;
    }
};

struct AttentionGrads {
    Tensor dq, dk, dv;
};

// The Op::FlashAttention backward arm (src/autograd.rs:3824-3916) with try_cudnn_sdpa_backward
// (:672-795): contiguous bf16 dQ/dK/dV; an fp32 upstream gradient is cast to bf16 instead of
// falling back to the materialising recompute (the reference bails out at :702-705).
inline Result<AttentionGrads> flash_attention_backward(const FlashAttentionNode& n, const Tensor& grad_out) {
    const auto& qs = n.query.shape();
    const auto& ks = n.key.shape();
    const int B = (int)qs[0], H = (int)qs[1], Sq = (int)qs[2], D = (int)qs[3], Sk = (int)ks[2];
    if (grad_out.shape() != n.output.shape()) return invalid("grad_out shape does not match the attention output");
    if (n.stats.dtype() != DType::F32 || n.stats.numel() != (int64_t)B * H * Sq)
        return invalid("saved Stats must be fp32 [B*H, Sq]");       // found by dtype + shape, :3877-3885
    Tensor g = grad_out;
    if (g.dtype() == DType::F32) {
        if (!g.is_contiguous()) return unsupported("strided fp32 grad_out");
        auto c = Tensor::empty(g.shape(), DType::BF16);
        if (!c.ok()) return c.error();
        const int rc = flame_attn_cast_f32_to_bf16(g.data(), c.value().data(), g.numel(), nullptr);
        if (rc != 0) return cuda_error("flame_attn_cast_f32_to_bf16", rc);
        g = c.value();
    } else if (g.dtype() != DType::BF16) {
        return invalid("grad_out must be BF16 or F32");
    }
    auto dq = Tensor::empty(n.query.shape(), DType::BF16);
    auto dk = Tensor::empty(n.key.shape(), DType::BF16);
    auto dv = Tensor::empty(n.value.shape(), DType::BF16);
    const size_t wsb = flame_attn_bwd_workspace_bytes(B, H, Sq, D);
    auto ws = Tensor::empty({(int64_t)wsb}, DType::U8);
    if (!dq.ok() || !dk.ok() || !dv.ok() || !ws.ok()) return cuda_error("hipMalloc", -1);
    Tensor m8;
    std::vector<int64_t> mst;
    if (n.mask) {
        auto pm = detail::prepare_mask(*n.mask, detail::Dims{B, H, Sq, Sk, D});
        if (!pm.ok()) return pm.error();
        m8 = pm.value().first;
        mst = pm.value().second;
    }
    int rc;
    if (n.dropout_p != 0.f) {
        rc = flame_attn_bwd_dropout_tiled_bf16(
            n.query.base(), n.key.base(), n.value.base(), n.output.base(), g.base(), n.stats.base(), dq.value().base(),
            dk.value().base(), dv.value().base(), B, H, Sq, Sk, D, n.scale, n.query.strides().data(), n.key.strides().data(),
            n.value.strides().data(), n.output.strides().data(), g.strides().data(), dq.value().strides().data(),
            dk.value().strides().data(), dv.value().strides().data(), n.query.offset(), n.key.offset(), n.value.offset(),
            n.output.offset(), g.offset(), 0, 0, 0, 0, n.causal ? 1 : 0, nullptr,
            n.mask ? static_cast<const uint8_t*>(m8.data()) : nullptr, n.mask ? mst.data() : nullptr, n.dropout_p, n.dropout_seed,
            n.draw_chunk_q, n.draw_chunk_kv, ws.value().data(), wsb, nullptr);
        if (rc != 0 && rc != FLAME_ATTN_ERR_UNSUPPORTED) return cuda_error("flame_attn_bwd_dropout_tiled_bf16", rc);
    } else {
        rc = flame_attn_bwd_bf16(
        n.query.base(), n.key.base(), n.value.base(), n.output.base(), g.base(), n.stats.base(), dq.value().base(),
        dk.value().base(), dv.value().base(), B, H, Sq, Sk, D, n.scale, n.query.strides().data(), n.key.strides().data(),
        n.value.strides().data(), n.output.strides().data(), g.strides().data(), dq.value().strides().data(),
        dk.value().strides().data(), dv.value().strides().data(), n.query.offset(), n.key.offset(), n.value.offset(),
        n.output.offset(), g.offset(), 0, 0, 0, 0, n.causal ? 1 : 0, nullptr,
        n.mask ? static_cast<const uint8_t*>(m8.data()) : nullptr, n.mask ? mst.data() : nullptr, ws.value().data(), wsb,
        nullptr);
    }
    if (rc == FLAME_ATTN_ERR_UNSUPPORTED) {
        // attention_backward_recompute (src/autograd.rs:801-848): the materialising backward for what the fused one
        // does not serve, here one band of query rows at a time
        const size_t wsm = flame_attn_materialised_workspace_bytes(B, H, Sq, Sk, D, D, 1);
        auto wm = Tensor::empty({(int64_t)wsm}, DType::U8);
        if (!wm.ok()) return wm.error();
        const int rm = flame_attn_bwd_materialised_bf16(
            n.query.base(), n.key.base(), n.value.base(), n.output.base(), g.base(), n.stats.base(), dq.value().base(),
            dk.value().base(), dv.value().base(), B, H, Sq, Sk, D, D, n.scale, n.query.strides().data(), n.key.strides().data(),
            n.value.strides().data(), n.output.strides().data(), g.strides().data(), dq.value().strides().data(),
            dk.value().strides().data(), dv.value().strides().data(), n.query.offset(), n.key.offset(), n.value.offset(),
            n.output.offset(), g.offset(), 0, 0, 0, 0, n.causal ? 1 : 0, nullptr,
            n.mask ? static_cast<const uint8_t*>(m8.data()) : nullptr, n.mask ? mst.data() : nullptr, n.dropout_p, n.dropout_seed,
            n.draw_chunk_q, n.draw_chunk_kv, wm.value().data(), wsm, nullptr);
        if (rm == FLAME_ATTN_ERR_UNSUPPORTED) return unsupported("flame_attn_bwd_materialised_bf16: layout not served (or rocBLAS missing)");
        if (rm != 0) return cuda_error("flame_attn_bwd_materialised_bf16", rm);
        return AttentionGrads{dq.value(), dk.value(), dv.value()};
    }
    if (rc != 0) return cuda_error("flame_attn_bwd_bf16", rc);
    return AttentionGrads{dq.value(), dk.value(), dv.value()};
}

inline Result<AttentionGrads> backward(const Tensor& attention_output, const Tensor& grad_out) {
    auto n = AutogradContext::find(attention_output);
    if (!n) return invalid("no FlashAttention node recorded for this tensor");
    return flash_attention_backward(*n, grad_out);
}

}  // namespace autograd

// ------------------------------------------------------------------------------------ sdpa
namespace sdpa {

inline Result<Tensor> forward_train(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask);

// sdpa::forward(q, k, v, mask) (src/sdpa.rs:85-102): routes to forward_train while taping
inline Result<Tensor> forward(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask = nullptr) {
    if (autograd::AutogradContext::is_recording() && (q.requires_grad || k.requires_grad || v.requires_grad))
        return forward_train(q, k, v, mask);
    auto r = detail::run_forward(q, k, v, mask, false, std::nullopt, false);
    if (!r.ok()) return r.error();
    return r.value().o;
}

// sdpa::forward_train (src/sdpa.rs:109-207): forward with Stats, then one Op::FlashAttention node;
// scale = 1/sqrt(D), causal = false.  Unlike the reference a mask keeps the O(S*D) path (the
// reference skips Stats for masked calls, :148-163).
inline Result<Tensor> forward_train(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask = nullptr) {
    auto r = detail::run_forward(q, k, v, mask, false, std::nullopt, true);
    if (!r.ok()) return r.error();
    Tensor o = r.value().o;
    o.requires_grad = true;
    autograd::FlashAttentionNode n;
    n.output_id = o.id();
    n.query = q; n.key = k; n.value = v; n.output = o; n.stats = r.value().stats;
    if (mask) n.mask = *mask;
    n.scale = 1.0f / std::sqrt((float)q.shape()[3]);
    n.causal = false;
    autograd::AutogradContext::record_op(std::move(n));
    return o;
}

// sdpa::forward_v4 (src/sdpa.rs:398-440): causal flag, optional scale, chunk sizes accepted and ignored
// (the fused kernel has no chunking knob)
inline Result<Tensor> forward_v4(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask, bool causal,
                                 std::optional<float> scale, std::optional<std::pair<size_t, size_t>> /*chunk*/ = std::nullopt) {
    auto r = detail::run_forward(q, k, v, mask, causal, scale, false);
    if (!r.ok()) return r.error();
    return r.value().o;
}

// sdpa::forward_with_bias(q, k, v, bias, scale) (src/sdpa.rs:232-328): additive float bias on the
// logits (T5-style relative position bias), softmax in fp32.  scale = None -> 1/sqrt(D); Some(s) ->
// multiply the scores by s.  bias: optional [B|1, H|1, Q, K], F32 or BF16.  Forward only, as in the
// reference; runs the fused kernel instead of materialising the fp32 score matrix.
inline Result<Tensor> forward_with_bias(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* bias,
                                        std::optional<float> scale) {
    auto dv = detail::validate(q, k, v, nullptr);
    if (!dv.ok()) return dv.error();
    const detail::Dims d = dv.value();
    if (!bias) return forward_v4(q, k, v, nullptr, false, scale);
    const auto& bs = bias->shape();
    if (bs.size() != 4) return invalid("bias must be 4D [B|1, H|1, Q, K]");
    if (!(bs[0] == d.B || bs[0] == 1) || !(bs[1] == d.H || bs[1] == 1) || bs[2] != d.Sq || bs[3] != d.Sk)
        return invalid("bias dims not broadcastable to [B,H,Q,K]");
    if (bias->dtype() != DType::F32 && bias->dtype() != DType::BF16) return invalid("bias must be F32 or BF16");
    for (const Tensor* t : {&q, &k, &v})
        if (!detail::abi_friendly(*t)) return unsupported("tensor view needs D stride 1 and 16-byte aligned rows; make it contiguous first");
    auto o = Tensor::empty({d.B, d.H, d.Sq, d.D}, DType::BF16);
    if (!o.ok()) return o.error();
    std::vector<int64_t> bst(4);
    const int64_t full[4] = {d.B, d.H, d.Sq, d.Sk};
    for (int i = 0; i < 4; ++i) bst[i] = (bs[i] == 1 && full[i] != 1) ? 0 : bias->strides()[i];
    const float sc = scale.value_or(1.0f / std::sqrt((float)d.D));
    const int rc = flame_attn_fwd_bias_bf16(q.base(), k.base(), v.base(), o.value().base(), nullptr, d.B, d.H, d.Sq, d.Sk, d.D, sc,
                                            q.strides().data(), k.strides().data(), v.strides().data(), o.value().strides().data(),
                                            q.offset(), k.offset(), v.offset(), 0, 0, bias->data(),
                                            bias->dtype() == DType::F32 ? FLAME_ATTN_DTYPE_F32 : FLAME_ATTN_DTYPE_BF16, bst.data(),
                                            nullptr, nullptr, nullptr);
    if (rc == FLAME_ATTN_ERR_UNSUPPORTED) return unsupported("flame_attn_fwd_bias_bf16: head dim or layout not built");
    if (rc != 0) return cuda_error("flame_attn_fwd_bias_bf16", rc);
    return o.value();
}

}  // namespace sdpa

// ------------------------------------------------------------------------------------ attention
namespace attention {

// lower-triangular keep-mask [1,1,Sq,Sk] (src/attention/sdpa.rs:11-34); the fused path does not need
// it (pass causal = true instead), it exists for callers that want the tensor
inline Result<Tensor> build_causal_mask(int64_t q_len, int64_t k_len) {
    std::vector<uint8_t> h((size_t)q_len * k_len);
    for (int64_t i = 0; i < q_len; ++i)
        for (int64_t j = 0; j < k_len; ++j) h[(size_t)i * k_len + j] = j <= i ? 1 : 0;
    return Tensor::from_host(h.data(), {1, 1, q_len, k_len}, DType::U8);
}

inline Result<Tensor> sdpa(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask = nullptr) {
    return flame::sdpa::forward(q, k, v, mask);
}
inline Result<Tensor> attend(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask = nullptr) {
    return flame::sdpa::forward(q, k, v, mask);
}
// attention::sdpa_with_bias(q, k, v, bias, scale) (src/attention/sdpa.rs:542-558)
inline Result<Tensor> sdpa_with_bias(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* bias,
                                     std::optional<float> scale) {
    return flame::sdpa::forward_with_bias(q, k, v, bias, scale);
}
// attention_impl(q, k, v, mask, causal, scale) (src/attention/sdpa.rs:395-458).  The reference
// rejects mask + causal together (:437-442); both are honoured here.
inline Result<Tensor> attention_impl(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask, bool causal,
                                     std::optional<float> scale) {
    return flame::sdpa::forward_v4(q, k, v, mask, causal, scale);
}

}  // namespace attention

// ------------------------------------------------------------------------------------ autograd_v4
namespace autograd_v4 {

enum class SdpaSave { SaveProbs, SaveLSE, Recompute };

struct SdpaConfig {                       // src/autograd_v4/ops/sdpa.rs:21-47
    bool causal = false;
    std::optional<float> scale;
    float dropout_p = 0.f;
    std::optional<uint64_t> dropout_seed;
    bool upcast_compute = true;
    std::optional<size_t> chunk_q, chunk_kv;
    SdpaSave save = SdpaSave::SaveLSE;
};

struct SdpaStats {                        // :56-65
    float fwd_ms = 0.f, bwd_ms = 0.f;
    uint64_t bytes_alloc = 0, bytes_saved = 0;
    uint32_t nan_inf_hits = 0, syncs = 0, recompute_blocks = 0;
};

// Debug hooks (:66-79, :1063-1074; the reference compiles them in under its `sdpa_debug` feature and
// hands them default-initialised statistics).  Registered once per process; while hooks are registered
// the forward and backward are timed with events, which costs one host synchronisation per call.
struct SdpaHooks {
    std::function<void(const SdpaConfig&, std::tuple<size_t, size_t, size_t, size_t>)> on_fwd_start;
    std::function<void(const SdpaStats&)> on_fwd_end;
    std::function<void()> on_bwd_start;
    std::function<void(const SdpaStats&)> on_bwd_end;
};
namespace detail_hooks {
inline std::unique_ptr<SdpaHooks>& slot() {
    static std::unique_ptr<SdpaHooks> h;
    return h;
}
inline std::mutex& guard() {
    static std::mutex m;
    return m;
}
}  // namespace detail_hooks
inline bool register_sdpa_hooks(SdpaHooks hooks) {          // false when hooks are already set (OnceCell::set)
    std::lock_guard<std::mutex> lk(detail_hooks::guard());
    if (detail_hooks::slot()) return false;
    detail_hooks::slot() = std::make_unique<SdpaHooks>(std::move(hooks));
    return true;
}
inline const SdpaHooks* debug_hooks() {
    std::lock_guard<std::mutex> lk(detail_hooks::guard());
    return detail_hooks::slot().get();
}
// wall time of everything enqueued on `stream` between construction and stop(), in ms
struct StreamTimer {
    explicit StreamTimer(hipStream_t s) : stream(s) {
        ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess && hipEventRecord(e0, stream) == hipSuccess;
    }
    float stop() {
        float ms = 0.f;
        if (ok && hipEventRecord(e1, stream) == hipSuccess && hipEventSynchronize(e1) == hipSuccess) hipEventElapsedTime(&ms, e0, e1);
        return ms;
    }
    ~StreamTimer() {
        if (e0) hipEventDestroy(e0);
        if (e1) hipEventDestroy(e1);
    }
    hipStream_t stream;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    bool ok = false;
};

struct SdpaCtx {                          // :80-96
    Tensor q, k, v, o;
    std::optional<Tensor> attn_mask;
    float scale = 0.f;
    SdpaSave save = SdpaSave::SaveLSE;
    bool causal = false;
    Tensor lse;                           // fp32 [B*H, Q]
    std::tuple<size_t, size_t, size_t, size_t> shapes;   // (B,H,Q,K)
    SdpaStats stats;
    float dropout_p = 0.f;                // :94-95
    std::optional<uint64_t> dropout_seed;
    std::pair<int, int> chunk_cfg{0, 0};  // (chunk_q, chunk_kv) the forward drew its dropout tiles with; 0 = whole axis
};

// ---- tape of the v4 engine (src/autograd_v4/graph.rs:12-94): nodes keyed by the output tensor's id,
//      in recording order; thread local.
struct Op {                               // the only variant on this path: Op::Sdpa
    std::shared_ptr<SdpaCtx> ctx;
    uint64_t q_id = 0, k_id = 0, v_id = 0;
};
struct GradNode {
    uint64_t id = 0;
    std::vector<uint64_t> parents;
    Op op;
};
struct Tape {
    std::unordered_map<uint64_t, std::shared_ptr<GradNode>> nodes;
    std::vector<uint64_t> order;
};
inline Tape& tape() {
    thread_local Tape t;
    return t;
}
// attach_backward_node / clear_tape (src/autograd_v4/ops/mod.rs:17-25)
inline void attach_backward_node(std::shared_ptr<GradNode> node) {
    tape().order.push_back(node->id);
    tape().nodes[node->id] = std::move(node);
}
inline void clear_tape() {
    tape().nodes.clear();
    tape().order.clear();
}

// Gradients (src/autograd_v4/gradients.rs:7-100): id -> fp32 gradient, accumulated on insert
class Gradients {
   public:
    Result<bool> accumulate(uint64_t id, const Tensor& grad) {
        if (grad.dtype() != DType::BF16 && grad.dtype() != DType::F32) return invalid("Gradients: gradient must be BF16 or F32");
        if (!grad.is_contiguous()) return unsupported("Gradients: gradient must be contiguous");
        auto it = map_.find(id);
        if (it == map_.end()) {
            auto acc = Tensor::empty(grad.shape(), DType::F32);
            if (!acc.ok()) return acc.error();
            int rc = flame_attn_fill(acc.value().data(), FLAME_ATTN_DTYPE_F32, 0.f, acc.value().numel(), nullptr);
            if (rc != 0) return cuda_error("flame_attn_fill", rc);
            it = map_.emplace(id, acc.value()).first;
        } else if (it->second.numel() != grad.numel()) {
            return invalid("Gradients: shape mismatch on accumulate");
        }
        const int rc = flame_attn_accumulate_f32(it->second.data(), grad.data(),
                                                 grad.dtype() == DType::F32 ? FLAME_ATTN_DTYPE_F32 : FLAME_ATTN_DTYPE_BF16,
                                                 grad.numel(), nullptr);
        if (rc != 0) return cuda_error("flame_attn_accumulate_f32", rc);
        return true;
    }
    const Tensor* get(uint64_t id) const {
        auto it = map_.find(id);
        return it == map_.end() ? nullptr : &it->second;
    }
    std::optional<Tensor> take(uint64_t id) {
        auto it = map_.find(id);
        if (it == map_.end()) return std::nullopt;
        Tensor t = it->second;
        map_.erase(it);
        return t;
    }
    void register_name(uint64_t id, std::string name) { names_[id] = std::move(name); }
    const std::string* name_for(uint64_t id) const {
        auto it = names_.find(id);
        return it == names_.end() ? nullptr : &it->second;
    }
    Result<bool> merge(const Gradients& other) {
        for (const auto& kv : other.map_) {
            auto r = accumulate(kv.first, kv.second);
            if (!r.ok()) return r.error();
        }
        for (const auto& kv : other.names_) names_.emplace(kv.first, kv.second);
        return true;
    }
    size_t size() const { return map_.size(); }

   private:
    std::unordered_map<uint64_t, Tensor> map_;
    std::unordered_map<uint64_t, std::string> names_;
};

// Seeds for calls that give none (the reference draws them from its global generator, src/rng/mod.rs:60-70 and
// src/autograd_v4/ops/sdpa.rs:120-124; deterministic after set_seed, though not the same stream as Rust's StdRng).
namespace rng {
inline std::mutex& guard() {
    static std::mutex m;
    return m;
}
inline uint64_t& state() {
    static uint64_t s = 0;
    return s;
}
inline void set_seed(uint64_t seed) {
    std::lock_guard<std::mutex> g(guard());
    state() = seed;
}
inline uint64_t next_u64() {          // SplitMix64
    std::lock_guard<std::mutex> g(guard());
    uint64_t z = (state() += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
}  // namespace rng

// sdpa_forward(q,k,v,mask,&cfg) -> (output, ctx) (:98-326).  SaveProbs would materialise the
// [B,H,Q,K] matrix and is refused rather than emulated.  Dropout (:110-124, :229-231) runs inside the fused
// kernels with the kept set the reference draws for the same seed: over the whole tensor, or, when the operator
// is chunked there (save = SaveLSE and chunk_q / chunk_kv smaller than the lengths, :180-199), per tile with the
// tile's seed (:600-602).  The attention itself is never chunked here: the chunk sizes only shape the kept set.
inline Result<std::pair<Tensor, SdpaCtx>> sdpa_forward(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask,
                                                       const SdpaConfig& cfg) {
    if (cfg.dropout_p < 0.f || cfg.dropout_p >= 1.f || cfg.dropout_p != cfg.dropout_p)
        return invalid("sdpa_forward: dropout_p=" + std::to_string(cfg.dropout_p) + " is out of range [0, 1)");
    std::optional<uint64_t> dropout_seed;
    if (cfg.dropout_p > 0.f) {
        dropout_seed = cfg.dropout_seed ? *cfg.dropout_seed : rng::next_u64();
    }
    // the reference chunks (and draws per tile) under SaveLSE only (:197-199)
    const int draw_cq = cfg.save == SdpaSave::SaveLSE && cfg.chunk_q ? (int)std::min<size_t>(*cfg.chunk_q, 1u << 30) : 0;
    const int draw_ck = cfg.save == SdpaSave::SaveLSE && cfg.chunk_kv ? (int)std::min<size_t>(*cfg.chunk_kv, 1u << 30) : 0;
    if (cfg.save == SdpaSave::SaveProbs) return unsupported("SaveProbs materialises [B,H,Q,K]; use SaveLSE");
    const SdpaHooks* hooks = debug_hooks();
    std::unique_ptr<StreamTimer> timer;
    if (hooks && q.shape().size() == 4 && k.shape().size() == 4) {
        if (hooks->on_fwd_start)
            hooks->on_fwd_start(cfg, {(size_t)q.shape()[0], (size_t)q.shape()[1], (size_t)q.shape()[2], (size_t)k.shape()[2]});
        timer = std::make_unique<StreamTimer>(nullptr);
    }
    // SaveLSE keeps O and the log-sum-exp for the backward; Recompute (:21-47) keeps neither and the backward
    // runs the forward once more to get them back (the outputs are deterministic, so it sees the same O).
    const bool keep = cfg.save != SdpaSave::Recompute;
    auto r = detail::run_forward(q, k, v, mask, cfg.causal, cfg.scale, keep, cfg.dropout_p, dropout_seed.value_or(0), draw_cq, draw_ck);
    if (!r.ok()) return r.error();
    SdpaCtx ctx;
    ctx.dropout_p = cfg.dropout_p;
    ctx.dropout_seed = dropout_seed;
    ctx.chunk_cfg = {draw_cq, draw_ck};
    ctx.q = q; ctx.k = k; ctx.v = v;
    if (keep) ctx.o = r.value().o;
    if (mask) ctx.attn_mask = *mask;
    ctx.scale = cfg.scale.value_or(1.0f / std::sqrt((float)q.shape()[3]));
    ctx.save = cfg.save;
    ctx.causal = cfg.causal;
    if (keep) ctx.lse = r.value().stats;
    ctx.shapes = {(size_t)q.shape()[0], (size_t)q.shape()[1], (size_t)q.shape()[2], (size_t)k.shape()[2]};
    ctx.stats.bytes_saved = keep ? (uint64_t)ctx.o.numel() * 2 + (uint64_t)ctx.lse.numel() * 4 : 0;
    ctx.stats.bytes_alloc = (uint64_t)r.value().o.numel() * 2 + (keep ? (uint64_t)ctx.lse.numel() * 4 : 0);   // what the forward allocated
    if (timer) {
        ctx.stats.fwd_ms = timer->stop();
        ctx.stats.syncs = 1;
        if (hooks->on_fwd_end) hooks->on_fwd_end(ctx.stats);
    }
    Tensor out = r.value().o;
    if (q.requires_grad || k.requires_grad || v.requires_grad) {     // record one Op::Sdpa node (:300-324)
        out.requires_grad = true;
        auto node = std::make_shared<GradNode>();
        node->id = out.id();
        node->op.ctx = std::make_shared<SdpaCtx>(ctx);
        node->op.q_id = q.id(); node->op.k_id = k.id(); node->op.v_id = v.id();
        for (const Tensor* t : {&q, &k, &v})
            if (t->requires_grad) node->parents.push_back(t->id());
        attach_backward_node(std::move(node));
    }
    return std::make_pair(out, ctx);
}

// sdpa_backward(&ctx, &grad_out) -> (dq, dk, dv) (:826-1009).  Gradients are bf16 here (the
// reference returns fp32 tensors from its fp32 tensor-op implementation).
inline Result<std::tuple<Tensor, Tensor, Tensor>> sdpa_backward(const SdpaCtx& ctx, const Tensor& grad_out) {
    autograd::FlashAttentionNode n;
    n.query = ctx.q; n.key = ctx.k; n.value = ctx.v; n.output = ctx.o; n.stats = ctx.lse;
    n.mask = ctx.attn_mask;
    n.scale = ctx.scale;
    n.causal = ctx.causal;
    n.dropout_p = ctx.dropout_p;
    n.dropout_seed = ctx.dropout_seed.value_or(0);
    n.draw_chunk_q = ctx.chunk_cfg.first;
    n.draw_chunk_kv = ctx.chunk_cfg.second;
    if (ctx.dropout_p > 0.f && !ctx.dropout_seed) return Error{Error::InvalidInput, "dropout seed required when dropout_p > 0"};
    if (ctx.save == SdpaSave::Recompute) {          // nothing was kept: O and the log-sum-exp come from one more forward
        auto f = detail::run_forward(ctx.q, ctx.k, ctx.v, ctx.attn_mask ? &*ctx.attn_mask : nullptr, ctx.causal, ctx.scale, true,
                                     ctx.dropout_p, ctx.dropout_seed.value_or(0));     // the same seed: the same kept set
        if (!f.ok()) return f.error();
        n.output = f.value().o;
        n.stats = f.value().stats;
    }
    const SdpaHooks* hooks = debug_hooks();
    std::unique_ptr<StreamTimer> timer;
    if (hooks) {
        if (hooks->on_bwd_start) hooks->on_bwd_start();
        timer = std::make_unique<StreamTimer>(nullptr);
    }
    auto g = autograd::flash_attention_backward(n, grad_out);
    if (!g.ok()) return g.error();
    if (timer) {
        SdpaStats st = ctx.stats;
        st.bwd_ms = timer->stop();
        st.syncs += 1;
        st.recompute_blocks = (uint32_t)(((std::get<2>(ctx.shapes) + 63) / 64) * ((std::get<3>(ctx.shapes) + 63) / 64));   // P tiles rebuilt per head
        if (hooks->on_bwd_end) hooks->on_bwd_end(st);
    }
    return std::make_tuple(g.value().dq, g.value().dk, g.value().dv);
}

// backward_v4(loss) (src/autograd_v4/ops/mod.rs:27-74): seed ones at the loss, walk the tape in reverse
// recording order, accumulate fp32 gradients for the parents that require them, clear the tape.  On this
// path the "loss" is an attention output itself (no other ops are taped), i.e. the seed is dL/dO = 1.
inline Result<Gradients> backward_v4(const Tensor& loss) {
    if (!loss.requires_grad) return Error{Error::InvalidInput, "backward_v4 called on tensor that does not require gradients"};
    Gradients grads;
    auto seed = Tensor::empty(loss.shape(), DType::F32);
    if (!seed.ok()) return seed.error();
    int rc = flame_attn_fill(seed.value().data(), FLAME_ATTN_DTYPE_F32, 1.0f, seed.value().numel(), nullptr);
    if (rc != 0) return cuda_error("flame_attn_fill", rc);
    auto acc = grads.accumulate(loss.id(), seed.value());
    if (!acc.ok()) return acc.error();
    const std::vector<uint64_t> order = tape().order;
    for (auto it = order.rbegin(); it != order.rend(); ++it) {
        auto nit = tape().nodes.find(*it);
        if (nit == tape().nodes.end()) continue;
        const std::shared_ptr<GradNode> node = nit->second;
        auto grad_out = grads.take(node->id);
        if (!grad_out) continue;                       // not reachable from the loss
        auto g = sdpa_backward(*node->op.ctx, *grad_out);
        if (!g.ok()) return g.error();
        const auto has = [&](uint64_t id) { return std::find(node->parents.begin(), node->parents.end(), id) != node->parents.end(); };
        if (has(node->op.q_id)) { auto r = grads.accumulate(node->op.q_id, std::get<0>(g.value())); if (!r.ok()) return r.error(); }
        if (has(node->op.k_id)) { auto r = grads.accumulate(node->op.k_id, std::get<1>(g.value())); if (!r.ok()) return r.error(); }
        if (has(node->op.v_id)) { auto r = grads.accumulate(node->op.v_id, std::get<2>(g.value())); if (!r.ok()) return r.error(); }
    }
    clear_tape();
    return grads;
}

}  // namespace autograd_v4

// ------------------------------------------------------------------------------------ streaming wrappers
// cuda_ops_bf16::sdpa_stream_bf16(q, k, v, mask, chunk, causal, scale) (src/cuda_ops_bf16.rs:1674-1684)
// and ops::attn::streaming_attn_bf16_fp32(q, k, v, StreamingAttnCfg) (src/ops/attn.rs:7-25, :327-598):
// the reference's host-looped / per-row streaming kernels.  Same arguments and checks; the chunk size is
// validated and otherwise ignored, the fused kernel streams K/V tiles by itself.
// JSONL telemetry of the streaming entry point (src/perf_telemetry.rs): one line per call appended to
// the file named by FLAME_SDPA_TELEMETRY_PATH, same keys in the same order.  The plan and autotune fields
// come from the library's launch-plan cache when the call went through flame_sdpa_chunked_bf16
// (contiguous tensors, no mask or a contiguous bf16 mask), as in src/cuda_ops_bf16.rs:2081-2127.

// staging::{SdpaAutotuneStats, sdpa_autotune_stats, reset_sdpa_autotune_stats, flush_sdpa_autotune_cache}
// (src/staging.rs:582-672): the counters of the launch-plan cache, same field names.
namespace staging {
using SdpaAutotuneStats = FlameSdpaAutotuneStats;
inline Result<SdpaAutotuneStats> sdpa_autotune_stats() {
    SdpaAutotuneStats raw{};
    const int rc = flame_sdpa_autotune_get_stats(&raw);
    if (rc != 0) return cuda_error("flame_sdpa_autotune_get_stats", rc);
    return raw;
}
inline Result<bool> reset_sdpa_autotune_stats() {
    const int rc = flame_sdpa_autotune_reset_stats();
    if (rc != 0) return cuda_error("flame_sdpa_autotune_reset_stats", rc);
    return true;
}
inline Result<bool> flush_sdpa_autotune_cache() {
    const int rc = flame_sdpa_autotune_flush_cache();
    if (rc != 0) return cuda_error("flame_sdpa_autotune_flush_cache", rc);
    return true;
}
}  // namespace staging

namespace perf_telemetry {
struct SdpaTelemetryRecord {                // :7-40
    size_t batch = 0, heads = 0, q_len = 0, k_len = 0, dh = 0, dv = 0, chunk_requested = 0;
    uint64_t tuned_q_chunk = 0, tuned_k_chunk = 0, plan_source = 0;
    size_t mask_heads = 0;
    bool has_mask = false, causal = false;
    uint64_t workspace_bytes = 0, stream_id = 0;
    double elapsed_ms = 0.0, tflops = 0.0;
    float scale = 0.f;
    uint64_t candidate_count = 0, best_time_ns = 0, autotune_env_forced = 0, autotune_clamped = 0, autotune_skipped = 0,
             autotune_fallback = 0, autotune_errors = 0, autotune_tuned = 0, cache_hits = 0, cache_misses = 0, cache_saved = 0,
             cache_loads = 0, cache_load_errors = 0, cache_entries = 0;
};
inline bool telemetry_enabled() {           // :60-66 (read once)
    static const bool on = [] {
        const char* p = std::getenv("FLAME_SDPA_TELEMETRY_PATH");
        return p && *p;
    }();
    return on;
}
namespace detail {
inline std::mutex& guard() {
    static std::mutex m;
    return m;
}
inline FILE* writer() {                     // :68-101: append, parent directory is the caller's business here
    static FILE* f = nullptr;
    if (!f) {
        const char* p = std::getenv("FLAME_SDPA_TELEMETRY_PATH");
        if (p && *p) f = std::fopen(p, "a");
    }
    return f;
}
inline unsigned long long now_ns() {
    return (unsigned long long)std::chrono::duration_cast<std::chrono::nanoseconds>(
               std::chrono::system_clock::now().time_since_epoch()).count();
}
}  // namespace detail
inline void log_sdpa_event(const SdpaTelemetryRecord& r) {          // :103-150
    if (!telemetry_enabled()) return;
    std::lock_guard<std::mutex> lk(detail::guard());
    FILE* f = detail::writer();
    if (!f) return;
    std::fprintf(f,
                 "{\"op\":\"sdpa_stream_bf16\",\"timestamp_ns\":%llu,\"batch\":%zu,\"heads\":%zu,\"q_len\":%zu,\"k_len\":%zu,"
                 "\"dh\":%zu,\"dv\":%zu,\"chunk_requested\":%zu,\"tuned_q_chunk\":%llu,\"tuned_k_chunk\":%llu,\"plan_source\":%llu,"
                 "\"mask_heads\":%zu,\"has_mask\":%d,\"causal\":%d,\"workspace_bytes\":%llu,\"stream_id\":%llu,\"elapsed_ms\":%.6f,"
                 "\"tflops\":%.6f,\"scale\":%.6f,\"candidate_count\":%llu,\"best_time_ns\":%llu,\"autotune_env_forced\":%llu,"
                 "\"autotune_clamped\":%llu,\"autotune_skipped\":%llu,\"autotune_fallback\":%llu,\"autotune_errors\":%llu,"
                 "\"autotune_tuned\":%llu,\"cache_hits\":%llu,\"cache_misses\":%llu,\"cache_saved\":%llu,\"cache_loads\":%llu,"
                 "\"cache_load_errors\":%llu,\"cache_entries\":%llu}\n",
                 detail::now_ns(), r.batch, r.heads, r.q_len, r.k_len, r.dh, r.dv, r.chunk_requested,
                 (unsigned long long)r.tuned_q_chunk, (unsigned long long)r.tuned_k_chunk, (unsigned long long)r.plan_source,
                 r.mask_heads, (int)r.has_mask, (int)r.causal, (unsigned long long)r.workspace_bytes,
                 (unsigned long long)r.stream_id, r.elapsed_ms, r.tflops, (double)r.scale,
                 (unsigned long long)r.candidate_count, (unsigned long long)r.best_time_ns,
                 (unsigned long long)r.autotune_env_forced, (unsigned long long)r.autotune_clamped,
                 (unsigned long long)r.autotune_skipped, (unsigned long long)r.autotune_fallback,
                 (unsigned long long)r.autotune_errors, (unsigned long long)r.autotune_tuned,
                 (unsigned long long)r.cache_hits, (unsigned long long)r.cache_misses, (unsigned long long)r.cache_saved,
                 (unsigned long long)r.cache_loads, (unsigned long long)r.cache_load_errors, (unsigned long long)r.cache_entries);
    std::fflush(f);
}
}  // namespace perf_telemetry

namespace cuda_ops_bf16 {
inline Result<Tensor> sdpa_stream_bf16(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask, size_t chunk,
                                       bool causal, std::optional<float> scale) {
    if (chunk == 0) return invalid("sdpa_stream_bf16: chunk must be > 0");
    // Contiguous BF16 tensors with no mask, or a contiguous BF16 mask [B, 1|H, Q, K], go through the chunked entry
    // point, which consults the launch-plan cache; every other layout takes the general forward.
    auto through_chunked = [&]() -> std::optional<Result<Tensor>> {
        if (q.shape().size() != 4 || k.shape().size() != 4 || v.shape().size() != 4) return std::nullopt;
        for (const Tensor* t : {&q, &k, &v})
            if (t->dtype() != DType::BF16 || !t->is_contiguous() || t->offset() != 0) return std::nullopt;
        const auto& qs = q.shape();
        const int64_t B = qs[0], H = qs[1], Q = qs[2], D = qs[3], K = k.shape()[2], Dv = v.shape()[3];
        if (k.shape()[0] != B || k.shape()[1] != H || k.shape()[3] != D || v.shape()[0] != B || v.shape()[1] != H ||
            v.shape()[2] != K)
            return std::nullopt;
        int mask_heads = 1;
        if (mask) {
            const auto& ms = mask->shape();
            if (mask->dtype() != DType::BF16 || !mask->is_contiguous() || mask->offset() != 0 || ms.size() != 4 || ms[0] != B ||
                (ms[1] != 1 && ms[1] != H) || ms[2] != Q || ms[3] != K)
                return std::nullopt;
            mask_heads = (int)ms[1];
        }
        auto o = Tensor::empty({B, H, Q, Dv}, DType::BF16);
        if (!o.ok()) return Result<Tensor>(o.error());
        const float sc = scale.value_or(1.0f / std::sqrt((float)D));
        const FlameAttnStatus st = flame_sdpa_chunked_bf16(q.base(), k.base(), v.base(), (int)B, (int)H, (int)Q, (int)K, (int)D, (int)Dv,
                                                           sc, (int)std::min<size_t>(chunk, 1u << 30), causal ? 1 : 0, mask_heads,
                                                           mask ? mask->base() : nullptr, o.value().base(), nullptr, 0, nullptr);
        if (st == FLAME_ATTN_STATUS_ERR_UNSUPPORTED) return std::nullopt;       // e.g. a head dim the kernels lack: general path reports it
        if (st != FLAME_ATTN_STATUS_OK) return Result<Tensor>(cuda_error("flame_sdpa_chunked_bf16", (int)st));
        return Result<Tensor>(o.value());
    };
    bool used_plan = false;
    auto run = [&]() -> Result<Tensor> {
        if (auto r = through_chunked()) {
            used_plan = true;
            return *r;
        }
        return flame::sdpa::forward_v4(q, k, v, mask, causal, scale);
    };
    if (!perf_telemetry::telemetry_enabled()) return run();
    autograd_v4::StreamTimer timer(nullptr);
    auto out = run();
    if (out.ok() && q.shape().size() == 4) {
        perf_telemetry::SdpaTelemetryRecord r;
        r.batch = (size_t)q.shape()[0]; r.heads = (size_t)q.shape()[1]; r.q_len = (size_t)q.shape()[2];
        r.k_len = (size_t)k.shape()[2]; r.dh = (size_t)q.shape()[3]; r.dv = (size_t)v.shape()[3];
        r.chunk_requested = chunk;
        r.tuned_q_chunk = 256; r.tuned_k_chunk = 64;          // the general forward: the largest tiles the kernels use
        if (used_plan) {
            if (auto st = staging::sdpa_autotune_stats(); st.ok()) {
                const auto& a = st.value();
                r.tuned_q_chunk = a.last_q_chunk; r.tuned_k_chunk = a.last_k_chunk; r.plan_source = a.last_plan_source;
                r.candidate_count = a.last_candidate_count; r.best_time_ns = a.last_best_time_ns;
                r.autotune_env_forced = a.env_forced; r.autotune_clamped = a.clamped; r.autotune_skipped = a.skipped;
                r.autotune_fallback = a.fallback; r.autotune_errors = a.errors; r.autotune_tuned = a.tuned;
                r.cache_hits = a.cache_hits; r.cache_misses = a.cache_misses; r.cache_saved = a.cache_saved;
                r.cache_loads = a.cache_loads; r.cache_load_errors = a.cache_load_errors; r.cache_entries = a.cache_entries;
            }
        }
        r.has_mask = mask != nullptr;
        r.mask_heads = mask && mask->shape().size() == 4 ? (size_t)mask->shape()[1] : 0;
        r.causal = causal;
        r.scale = scale.value_or(1.0f / std::sqrt((float)q.shape()[3]));
        r.elapsed_ms = timer.stop();
        const double pairs = (double)r.batch * r.heads * r.q_len * r.k_len * (causal ? 0.5 : 1.0);
        r.tflops = r.elapsed_ms > 0 ? 4.0 * pairs * (double)r.dh / (r.elapsed_ms * 1e-3) / 1e12 : 0.0;
        perf_telemetry::log_sdpa_event(r);
    }
    return out;
}

// src/cuda_ops_bf16.rs:49-52, :1686-1695: the reference lets the caller bring the device scratch of its host-looped
// kernels (fp32 logits of one chunk and running rows).  The fused forward keeps those in registers and LDS: a
// workspace is accepted, checked for consistency and left untouched.
struct SdpaWorkspace {
    void* ptr = nullptr;
    uint64_t bytes = 0;
};
inline Result<Tensor> sdpa_stream_bf16_with_workspace(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* mask, size_t chunk,
                                                      bool causal, std::optional<float> scale, std::optional<SdpaWorkspace> workspace) {
    if (workspace && workspace->bytes > 0 && !workspace->ptr) return invalid("sdpa_stream_bf16: workspace pointer is null");
    return sdpa_stream_bf16(q, k, v, mask, chunk, causal, scale);
}
}  // namespace cuda_ops_bf16

namespace ops {
namespace attn {
// src/ops/attn.rs:327-598.  The reference's function plans a query chunk whose fp32 scratch (chunk x K logits plus
// running rows, :72-84) fits a budget taken from free device memory and steps down a list of chunks when a launch
// fails (:113-209, :453-592).  The fused forward keeps that scratch in registers and LDS and runs the same launch
// whatever the chunk, so nothing is planned, budgeted or retried here: the chunk is validated (0 is an error, as
// there) and otherwise has no effect.
// Beyond the reference: a keep-mask is taken (bf16, 1 = keep; the reference's function refuses one, :366-370,
// although its test passes one, tests/streaming_attn.rs:413-489), and the three tensors may be strided views and
// have key lengths of their own.
struct StreamingAttnCfg {                                     // :8-25
    float scale = 1.0f;
    size_t chunk_size = 2048;
    bool causal = false;
    const Tensor* mask = nullptr;
};

inline Result<Tensor> streaming_attn_bf16_fp32(const Tensor& q, const Tensor& k, const Tensor& v, const StreamingAttnCfg& cfg) {
    if (cfg.chunk_size == 0) return invalid("streaming attention chunk_size must be > 0");
    if (q.dtype() != DType::BF16 || k.dtype() != DType::BF16 || v.dtype() != DType::BF16)
        return invalid("streaming attention expects BF16 tensors");
    if (q.shape().size() != 4 || k.shape().size() != 4 || v.shape().size() != 4) return invalid("expected 4D tensors");
    if (q.shape()[3] != k.shape()[3]) return invalid("head dimensions for Q and K differ");
    return cuda_ops_bf16::sdpa_stream_bf16(q, k, v, cfg.mask, cfg.chunk_size, cfg.causal, cfg.scale);
}
}  // namespace attn
}  // namespace ops

// ------------------------------------------------------------------------------------ input preparation
// Counterparts of the reference's rope_fused_bf16 / rope_fused_bf16_f32pe (src/bf16_ops.rs:476-582,
// x [B,H,N,D], tables [1,1,N,D/2]) and of its per-head RMSNorm (src/norm.rs:1090-1092,
// x * weight / sqrt(mean(x^2) + eps) over the last dim), plus the fused form that reads the
// projection output [B,N,H,D] and returns the normalised, rotated [B,H,N,D] tensor in one pass.
namespace bf16_ops {
namespace detail_prep {
inline Result<Tensor> run(const Tensor& x_bhnd, const Tensor* weight, const Tensor* cos, const Tensor* sin, float eps,
                          bool apply_norm, const char* who) {
    if (x_bhnd.shape().size() != 4) return invalid(std::string(who) + ": expected 4D [B,H,N,D]");
    if (x_bhnd.dtype() != DType::BF16) return invalid(std::string(who) + ": expects BF16");
    const auto& sh = x_bhnd.shape();
    const int64_t B = sh[0], H = sh[1], N = sh[2], D = sh[3];
    int tdt = FLAME_ATTN_DTYPE_BF16;
    if ((cos == nullptr) != (sin == nullptr)) return invalid(std::string(who) + ": cos and sin go together");
    if (cos) {
        if (cos->dtype() != sin->dtype() || (cos->dtype() != DType::BF16 && cos->dtype() != DType::F32))
            return invalid(std::string(who) + ": cos/sin must both be BF16 or both F32");
        if (cos->numel() != N * (D / 2) || sin->numel() != N * (D / 2) || !cos->is_contiguous() || !sin->is_contiguous())
            return invalid(std::string(who) + ": cos/sin must be contiguous [1,1,N,D/2]");
        tdt = cos->dtype() == DType::F32 ? FLAME_ATTN_DTYPE_F32 : FLAME_ATTN_DTYPE_BF16;
    }
    if (weight && (weight->dtype() != DType::BF16 || weight->numel() != D)) return invalid(std::string(who) + ": weight must be BF16 [D]");
    auto y = Tensor::empty({B, H, N, D}, DType::BF16);
    if (!y.ok()) return y.error();
    const int rc = flame_attn_prep_rmsnorm_rope_bf16(x_bhnd.base(), weight ? weight->data() : nullptr, cos ? cos->data() : nullptr,
                                                     sin ? sin->data() : nullptr, tdt, y.value().base(), (int)B, (int)H, (int)N,
                                                     (int)D, eps, apply_norm ? 1 : 0, x_bhnd.strides().data(),
                                                     y.value().strides().data(), x_bhnd.offset(), 0, nullptr);
    if (rc == FLAME_ATTN_ERR_UNSUPPORTED) return unsupported(std::string(who) + ": head dim or layout not built");
    if (rc == FLAME_ATTN_ERR_INVALID) return invalid(std::string(who) + ": bad arguments");
    if (rc != 0) return cuda_error(who, rc);
    return y.value();
}
}  // namespace detail_prep

inline Result<Tensor> rope_fused_bf16(const Tensor& x, const Tensor& cos, const Tensor& sin) {
    if (cos.dtype() != DType::BF16 || sin.dtype() != DType::BF16) return invalid("rope_fused_bf16: cos/sin must be BF16");
    return detail_prep::run(x, nullptr, &cos, &sin, 0.f, false, "rope_fused_bf16");
}
inline Result<Tensor> rope_fused_bf16_f32pe(const Tensor& x, const Tensor& cos, const Tensor& sin) {
    if (cos.dtype() != DType::F32 || sin.dtype() != DType::F32) return invalid("rope_fused_bf16_f32pe: cos/sin must be F32");
    return detail_prep::run(x, nullptr, &cos, &sin, 0.f, false, "rope_fused_bf16_f32pe");
}
}  // namespace bf16_ops

namespace norm {
// RMSNorm over the last (head) dim of a 4-D tensor.
inline Result<Tensor> rms_norm(const Tensor& x, const Tensor* weight, float eps) {
    return bf16_ops::detail_prep::run(x, weight, nullptr, nullptr, eps, true, "rms_norm");
}
}  // namespace norm

namespace attention {
// x: projection output [B,N,H,D] (any strides over B, N, H).  Returns rope(rms_norm(x) * weight) as
// contiguous [B,H,N,D]; weight and the tables are optional.
inline Result<Tensor> prep_qk(const Tensor& x_bnhd, const Tensor* weight, const Tensor* cos, const Tensor* sin, float eps = 1e-6f) {
    if (x_bnhd.shape().size() != 4) return invalid("prep_qk: expected 4D [B,N,H,D]");
    return bf16_ops::detail_prep::run(x_bnhd.permute({0, 2, 1, 3}), weight, cos, sin, eps, true, "prep_qk");
}
}  // namespace attention

// ------------------------------------------------------------------------------------ SageAttention
// Builder-style API of the reference (src/sage_attention.rs:21-65).  `scale` is the softmax scale
// (default 1/sqrt(D)); the reference's field of the same name is a divisor defaulting to sqrt(D)
// (:108, :588), i.e. the same default arithmetic.  int8 Q/K per block, mean-smoothed K.
//
// forward(q, k, v, attention_mask): attention_mask is ADDED to the scores before the softmax, as the
// reference does (:126-131): F32 or BF16, [B|1, H|1, Sq, Sk], -inf excludes a position.
// forward_saving(...) also returns what the reference records for its backward (:134-150): the query, the
// smoothed key and the value.  The materialised attention weights it saves as well are not produced here;
// sage_attention_backward recomputes them tile by tile.
struct SageSaved {
    Tensor output, query, key_smoothed, value;
    float scale = 0.f;
    bool causal = false;
};

class SageAttention {
   public:
    SageAttention() = default;
    SageAttention with_scale(float softmax_scale) const { auto s = *this; s.scale_ = softmax_scale; return s; }
    SageAttention with_causal(bool causal) const { auto s = *this; s.causal_ = causal; return s; }
    SageAttention with_smoothing(bool on) const { auto s = *this; s.smooth_k_ = on; return s; }

    Result<Tensor> forward(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* attention_mask = nullptr) const {
        auto r = run(q, k, v, attention_mask, false);
        if (!r.ok()) return r.error();
        return r.value().output;
    }
    Result<SageSaved> forward_saving(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* attention_mask = nullptr) const {
        return run(q, k, v, attention_mask, true);
    }

   private:
    Result<SageSaved> run(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor* bias, bool save) const {
        auto dv = detail::validate(q, k, v, nullptr);
        if (!dv.ok()) return dv.error();
        const detail::Dims d = dv.value();
        for (const Tensor* t : {&q, &k, &v})
            if (!detail::abi_friendly(*t)) return unsupported("tensor view needs D stride 1 and 16-byte aligned rows");
        std::vector<int64_t> bst(4, 0);
        if (bias) {
            const auto& bs = bias->shape();
            if (bs.size() != 4) return invalid("attention_mask must be 4D [B|1, H|1, Q, K]");
            if (!(bs[0] == d.B || bs[0] == 1) || !(bs[1] == d.H || bs[1] == 1) || bs[2] != d.Sq || bs[3] != d.Sk)
                return invalid("attention_mask dims not broadcastable to [B,H,Q,K]");
            if (bias->dtype() != DType::F32 && bias->dtype() != DType::BF16) return invalid("attention_mask must be F32 or BF16 (it is added to the scores)");
            const int64_t full[4] = {d.B, d.H, d.Sq, d.Sk};
            for (int i = 0; i < 4; ++i) bst[i] = (bs[i] == 1 && full[i] != 1) ? 0 : bias->strides()[i];
        }
        const int64_t nqb = (d.Sq + 127) / 128, nkb = (d.Sk + 63) / 64;
        // the quantiser writes rows of 64 (head dims up to 64) or 128 elements, zero beyond the head dim
        const int64_t dr = d.D <= 64 ? 64 : 128;
        auto qi8 = Tensor::empty({d.B, d.H, d.Sq, dr}, DType::I8);
        auto ki8 = Tensor::empty({d.B, d.H, d.Sk, dr}, DType::I8);
        auto sq = Tensor::empty({d.B, d.H, nqb}, DType::F32);
        auto sk = Tensor::empty({d.B, d.H, nkb}, DType::F32);
        auto km = Tensor::empty({d.B, d.H, dr}, DType::F32);
        auto o = Tensor::empty({d.B, d.H, d.Sq, d.D}, DType::BF16);
        if (!qi8.ok() || !ki8.ok() || !sq.ok() || !sk.ok() || !km.ok() || !o.ok()) return cuda_error("hipMalloc", -1);
        Tensor ks;
        if (save) {
            auto t = Tensor::empty({d.B, d.H, d.Sk, dr}, DType::BF16);
            if (!t.ok()) return t.error();
            ks = t.value().narrow_last(d.D);
        }
        int rc = flame_sage_quant_qk_int8_ks(q.base(), k.base(), d.B, d.H, d.Sq, d.Sk, d.D, q.strides().data(), k.strides().data(),
                                             q.offset(), k.offset(), smooth_k_ ? 1 : 0, qi8.value().data(), ki8.value().data(),
                                             sq.value().data(), sk.value().data(), km.value().data(), save ? ks.data() : nullptr,
                                             nullptr);
        if (rc == FLAME_ATTN_ERR_UNSUPPORTED) return unsupported("flame_sage_quant_qk_int8: head dim or layout not built");
        if (rc != 0) return cuda_error("flame_sage_quant_qk_int8", rc);
        const float sc = scale_.value_or(1.0f / std::sqrt((float)d.D));
        rc = flame_sage_attn_fwd_bias_int8(qi8.value().data(), ki8.value().data(), sq.value().data(), sk.value().data(), v.base(),
                                           o.value().base(), nullptr, d.B, d.H, d.Sq, d.Sk, d.D, sc, v.strides().data(),
                                           o.value().strides().data(), v.offset(), 0, causal_ ? 1 : 0, nullptr,
                                           bias ? bias->data() : nullptr,
                                           bias && bias->dtype() == DType::BF16 ? FLAME_ATTN_DTYPE_BF16 : FLAME_ATTN_DTYPE_F32,
                                           bias ? bst.data() : nullptr, nullptr);
        if (rc != 0) return cuda_error("flame_sage_attn_fwd_int8", rc);
        return SageSaved{o.value(), q, ks, v, sc, causal_};
    }

    std::optional<float> scale_;
    bool causal_ = false;
    bool smooth_k_ = true;
};

// sage_attention_backward (src/sage_attention.rs:470-505): the reference's backward of its Sage operator is
// "standard attention backward" on (query, key_smoothed, value), ignoring the quantisation, from the
// materialised attention weights it saved.  The same gradients here without that [B,H,Sq,Sk] tensor: one bf16
// forward recomputes O and the log-sum-exp of (query, key_smoothed, value), then the tile-recompute backward
// runs.  `scale` is the softmax scale (a multiplier; the reference passes its divisor).  As in the reference
// the key gradient is the one with respect to the smoothed key.
inline Result<autograd::AttentionGrads> sage_attention_backward(const Tensor& grad_output, const Tensor& query,
                                                                const Tensor& key_smoothed, const Tensor& value, float scale,
                                                                bool causal) {
    auto f = detail::run_forward(query, key_smoothed, value, nullptr, causal, scale, true);
    if (!f.ok()) return f.error();
    autograd::FlashAttentionNode n;
    n.query = query; n.key = key_smoothed; n.value = value;
    n.output = f.value().o; n.stats = f.value().stats;
    n.scale = scale; n.causal = causal;
    return autograd::flash_attention_backward(n, grad_output);
}
inline Result<autograd::AttentionGrads> sage_attention_backward(const SageSaved& s, const Tensor& grad_output) {
    return sage_attention_backward(grad_output, s.query, s.key_smoothed, s.value, s.scale, s.causal);
}

}  // namespace flame
