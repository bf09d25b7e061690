// Test harness, not part of the library: a caller-side activation offload pool in the shape of the reference's
// (src/activation_offload.rs:84-96, :291-304, :365-775), used by host_api_test.cpp to drive the two FP8 entry points
// of the library (flame_bf16_to_fp8 / flame_fp8_to_bf16) the way that pool drives them: on a transfer stream of its
// own, between pinned host buffers and device staging buffers, with the saved set of one attention call.
#pragma once

#include "../../flame_amd/host/flame_host.hpp"

namespace flame {
// ------------------------------------------------------------------------------------ activation offload
// Saved activations pushed to pinned host memory in the forward and pulled back in the backward
// (src/activation_offload.rs).  One transfer stream of the pool's own (non-blocking, default priority), one pinned
// buffer and two events per slot, no host synchronisation in push or pull:
//   push: record done[slot] on the default stream, the transfer stream waits for it, then (FP8: quantise into the
//         slot's device staging buffer, then) copy device -> host on the transfer stream;
//   pull: copy host -> device on the transfer stream (same-stream order puts it after the push's copy; FP8: into
//         the staging buffer, then dequantise into the new tensor), record ready[slot] there, the default stream
//         waits for it.
// Slots are handed out from a stack (LIFO, the order the backward consumes them); a full pool refuses the push;
// clear() frees every slot and makes the handles issued so far stale.  The pushed tensor is kept alive until its
// slot is drained.  FP8 halves host memory and link traffic with the reference's fixed scale 8/448 (:543-549).
namespace activation_offload {

enum class OffloadCompression { None, FP8 };

class OffloadHandle {                      // :291-304
   public:
    size_t slot() const { return slot_; }

   private:
    friend class ActivationOffloadPool;
    size_t slot_ = 0;
    uint64_t epoch_ = 0;
};

class ActivationOffloadPool {
   public:
    ActivationOffloadPool(const ActivationOffloadPool&) = delete;
    ActivationOffloadPool& operator=(const ActivationOffloadPool&) = delete;

    // :365-428
    static Result<std::unique_ptr<ActivationOffloadPool>> create(size_t num_slots, size_t max_bytes, OffloadCompression compression) {
        if (num_slots == 0) return invalid("ActivationOffloadPool::new: num_slots must be > 0");
        if (max_bytes == 0) return invalid("ActivationOffloadPool::new: max_bytes must be > 0");
        std::unique_ptr<ActivationOffloadPool> p(new ActivationOffloadPool());
        p->compression_ = compression;
        p->slot_bytes_ = max_bytes;
        const size_t host_buf_bytes = compression == OffloadCompression::FP8 ? (max_bytes + 1) / 2 : max_bytes;
        hipError_t e = hipStreamCreateWithFlags(&p->transfer_, hipStreamNonBlocking);
        if (e != hipSuccess) return cuda_error("hipStreamCreateWithFlags", (int)e);
        for (size_t i = 0; i < num_slots; ++i) {
            void* h = nullptr;
            if ((e = hipHostMalloc(&h, host_buf_bytes, hipHostMallocDefault)) != hipSuccess) return cuda_error("hipHostMalloc", (int)e);
            p->host_.push_back(h);
            hipEvent_t d, r;
            if ((e = hipEventCreateWithFlags(&d, hipEventDisableTiming)) != hipSuccess) return cuda_error("hipEventCreate", (int)e);
            p->done_.push_back(d);
            if ((e = hipEventCreateWithFlags(&r, hipEventDisableTiming)) != hipSuccess) return cuda_error("hipEventCreate", (int)e);
            p->ready_.push_back(r);
            if (compression == OffloadCompression::FP8) {
                void* g = nullptr;
                if ((e = hipMalloc(&g, host_buf_bytes)) != hipSuccess) return cuda_error("hipMalloc", (int)e);
                p->staging_.push_back(g);
            }
        }
        p->meta_.resize(num_slots);
        p->pushed_.assign(num_slots, false);
        p->keep_alive_.resize(num_slots);
        for (size_t i = num_slots; i-- > 0;) p->free_stack_.push_back(i);     // slot 0 on top
        return p;
    }
    ~ActivationOffloadPool() {
        if (transfer_) (void)hipStreamSynchronize(transfer_);
        for (void* g : staging_) (void)hipFree(g);
        for (void* h : host_) (void)hipHostFree(h);
        for (hipEvent_t e : done_) (void)hipEventDestroy(e);
        for (hipEvent_t e : ready_) (void)hipEventDestroy(e);
        if (transfer_) (void)hipStreamDestroy(transfer_);
    }

    size_t num_slots() const { return host_.size(); }                        // :431-434
    size_t slot_bytes() const { return slot_bytes_; }                        // :437-440
    size_t host_bytes() const {                                              // :443-450
        return (compression_ == OffloadCompression::FP8 ? (slot_bytes_ + 1) / 2 : slot_bytes_) * host_.size();
    }
    size_t in_flight() const { return (size_t)std::count(pushed_.begin(), pushed_.end(), true); }   // :453-455

    // :465-617
    Result<OffloadHandle> push(const Tensor& t) {
        if (!t.defined()) return invalid("ActivationOffloadPool::push: tensor is empty");
        if (t.dtype() != DType::BF16 && t.dtype() != DType::F32)
            return unsupported("ActivationOffloadPool::push: dtype not supported (BF16/F32 only)");
        if (!t.is_contiguous()) return unsupported("ActivationOffloadPool::push: tensor is a strided view");
        const size_t numel = (size_t)t.numel(), bytes = numel * dtype_size(t.dtype());
        if (bytes == 0) return invalid("ActivationOffloadPool::push: tensor is empty");
        if (bytes > slot_bytes_)
            return invalid("ActivationOffloadPool::push: tensor " + std::to_string(bytes) + " bytes exceeds slot capacity " +
                           std::to_string(slot_bytes_) + " bytes");
        if (compression_ == OffloadCompression::FP8 && t.dtype() != DType::BF16)
            return unsupported("FP8 compression only supports BF16 activations");
        if (free_stack_.empty())
            return Error{Error::InvalidOperation, "ActivationOffloadPool full: " + std::to_string(host_.size()) +
                                                       " slots all in-flight. Increase num_slots."};
        const size_t slot = free_stack_.back();
        free_stack_.pop_back();
        auto fail = [&](const char* what, int code) {
            free_stack_.push_back(slot);
            return cuda_error(std::string("activation offload push: ") + what, code);
        };
        hipError_t e = hipEventRecord(done_[slot], nullptr);                  // the producer's progress on the default stream
        if (e != hipSuccess) return fail("event record", (int)e);
        if ((e = hipStreamWaitEvent(transfer_, done_[slot], 0)) != hipSuccess) return fail("stream wait", (int)e);
        SlotMeta m{t.shape(), t.dtype(), bytes, bytes, numel, 0.f};
        if (compression_ == OffloadCompression::None) {
            if ((e = hipMemcpyAsync(host_[slot], t.data(), bytes, hipMemcpyDeviceToHost, transfer_)) != hipSuccess)
                return fail("DtoH failed", (int)e);
        } else {
            const float scale = 8.0f / 448.0f, inv_scale = 1.0f / scale;      // activations in [-8, 8] assumed (:543-549)
            int rc = flame_bf16_to_fp8(t.data(), staging_[slot], inv_scale, numel, transfer_);
            if (rc != 0) return fail("bf16_to_fp8 failed", rc);
            if ((e = hipMemcpyAsync(host_[slot], staging_[slot], numel, hipMemcpyDeviceToHost, transfer_)) != hipSuccess)
                return fail("FP8 DtoH failed", (int)e);
            m.stored_bytes = numel;
            m.fp8_scale = scale;
        }
        meta_[slot] = std::move(m);
        pushed_[slot] = true;
        keep_alive_[slot] = t;
        OffloadHandle h;
        h.slot_ = slot;
        h.epoch_ = epoch_;
        return h;
    }

    // :619-737
    Result<Tensor> pull(OffloadHandle h) {
        if (h.epoch_ != epoch_)
            return Error{Error::InvalidOperation, "ActivationOffloadPool::pull: handle epoch " + std::to_string(h.epoch_) +
                                                       " is stale (current " + std::to_string(epoch_) + ")"};
        if (h.slot_ >= host_.size())
            return Error{Error::InvalidOperation, "ActivationOffloadPool::pull: slot " + std::to_string(h.slot_) + " out of range"};
        if (!pushed_[h.slot_])
            return Error{Error::InvalidOperation, "ActivationOffloadPool::pull: slot " + std::to_string(h.slot_) +
                                                       " is idle, expected pushed (double pull?)"};
        const size_t slot = h.slot_;
        const SlotMeta& m = *meta_[slot];
        auto out = Tensor::empty(m.shape, m.dtype);
        if (!out.ok()) return out.error();
        hipError_t e;
        if (compression_ == OffloadCompression::None) {
            e = hipMemcpyAsync(out.value().data(), host_[slot], m.stored_bytes, hipMemcpyHostToDevice, transfer_);
            if (e != hipSuccess) return cuda_error("activation offload pull: HtoD failed", (int)e);
        } else {
            e = hipMemcpyAsync(staging_[slot], host_[slot], m.stored_bytes, hipMemcpyHostToDevice, transfer_);
            if (e != hipSuccess) return cuda_error("activation offload pull: HtoD failed", (int)e);
            int rc = flame_fp8_to_bf16(staging_[slot], out.value().data(), m.fp8_scale, m.numel, transfer_);
            if (rc != 0) return cuda_error("activation offload pull: fp8_to_bf16 failed", rc);
        }
        if ((e = hipEventRecord(ready_[slot], transfer_)) != hipSuccess) return cuda_error("activation offload pull: event record", (int)e);
        if ((e = hipStreamWaitEvent(nullptr, ready_[slot], 0)) != hipSuccess) return cuda_error("activation offload pull: stream wait", (int)e);
        meta_[slot].reset();
        pushed_[slot] = false;
        keep_alive_[slot] = Tensor();
        free_stack_.push_back(slot);
        return out;
    }

    // :742-761: every slot idle again, handles issued so far stale; no host synchronisation (call synchronize()
    // first if a copy may still be reading a pinned buffer)
    void clear() {
        for (size_t i = 0; i < host_.size(); ++i) {
            pushed_[i] = false;
            meta_[i].reset();
            keep_alive_[i] = Tensor();
        }
        free_stack_.clear();
        for (size_t i = host_.size(); i-- > 0;) free_stack_.push_back(i);
        if (++epoch_ == 0) epoch_ = 1;
    }
    Result<bool> synchronize() {
        hipError_t e = hipStreamSynchronize(transfer_);
        if (e != hipSuccess) return cuda_error("hipStreamSynchronize", (int)e);
        return true;
    }

   private:
    ActivationOffloadPool() = default;
    struct SlotMeta {                        // :269-281
        std::vector<int64_t> shape;
        DType dtype;
        size_t bytes, stored_bytes, numel;
        float fp8_scale;                     // 0 = not compressed
    };
    OffloadCompression compression_ = OffloadCompression::None;
    size_t slot_bytes_ = 0;
    uint64_t epoch_ = 1;
    hipStream_t transfer_ = nullptr;
    std::vector<void*> host_, staging_;
    std::vector<hipEvent_t> done_, ready_;
    std::vector<std::optional<SlotMeta>> meta_;
    std::vector<bool> pushed_;
    std::vector<Tensor> keep_alive_;
    std::vector<size_t> free_stack_;
};

}  // namespace activation_offload

// The saved set of one attention call through the pool: Q, K, V and O leave the device (pushed in that order),
// the log-sum-exp rows stay (fp32, 1/256 of the bytes at D = 128; an FP8 pool takes bf16 only, :536-541).
// restore_saved pulls in reverse order, as the slots' stack expects, and gives the context the backward takes.
namespace autograd_v4 {
struct OffloadedSdpaCtx {
    SdpaCtx rest;                                              // q, k, v, o undefined while offloaded
    activation_offload::OffloadHandle q, k, v, o;
};
inline Result<OffloadedSdpaCtx> offload_saved(const SdpaCtx& ctx, activation_offload::ActivationOffloadPool& pool) {
    OffloadedSdpaCtx off;
    off.rest = ctx;
    const Tensor* src[4] = {&ctx.q, &ctx.k, &ctx.v, &ctx.o};
    activation_offload::OffloadHandle* dst[4] = {&off.q, &off.k, &off.v, &off.o};
    for (int i = 0; i < 4; ++i) {
        if (i == 3 && ctx.save == SdpaSave::Recompute) break;  // no O was kept
        auto h = pool.push(*src[i]);
        if (!h.ok()) {
            for (int j = i; j-- > 0;) (void)pool.pull(*dst[j]);   // give the slots back
            return h.error();
        }
        *dst[i] = h.value();
    }
    off.rest.q = off.rest.k = off.rest.v = Tensor();
    if (ctx.save != SdpaSave::Recompute) off.rest.o = Tensor();
    return off;
}
inline Result<SdpaCtx> restore_saved(const OffloadedSdpaCtx& off, activation_offload::ActivationOffloadPool& pool) {
    SdpaCtx ctx = off.rest;
    if (ctx.save != SdpaSave::Recompute) {
        auto o = pool.pull(off.o);
        if (!o.ok()) return o.error();
        ctx.o = o.value();
    }
    auto v = pool.pull(off.v);
    if (!v.ok()) return v.error();
    auto k = pool.pull(off.k);
    if (!k.ok()) return k.error();
    auto q = pool.pull(off.q);
    if (!q.ok()) return q.error();
    ctx.q = q.value(); ctx.k = k.value(); ctx.v = v.value();
    return ctx;
}
}  // namespace autograd_v4

}  // namespace flame
