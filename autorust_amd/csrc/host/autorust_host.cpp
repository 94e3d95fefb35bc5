// Implementation of the C++ mirror of the reference's attention interface (autorust_host.h).
// Everything computes through libarhip's C ABI; nothing here touches HIP directly.
#include "autorust_host.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace autorust {

const char *name(AttentionKind k)
{
    switch (k) {
    case AttentionKind::Sdpa: return "sdpa";
    case AttentionKind::Flash: return "flash";
    default: return "sage";
    }
}

AttentionKind attention_kind_from_str(const std::string &s)
{
    if (s == "sdpa") return AttentionKind::Sdpa;
    if (s == "sage") return AttentionKind::Sage;
    return AttentionKind::Flash;  // the default, also for unknown values (settings.rs:209-213)
}

static bool env_flag(const char *n, bool dflt)
{
    const char *v = getenv(n);
    if (!v || !*v) return dflt;
    return !(v[0] == '0' || v[0] == 'f' || v[0] == 'F' || v[0] == 'n' || v[0] == 'N');
}

Settings Settings::from_env()
{
    Settings s;
    if (const char *a = getenv("AUTORUST_ATTN")) s.attention = attention_kind_from_str(a);
    s.tensor_cores = env_flag("AUTORUST_TENSOR_CORES", env_flag("AUTORUST_TC", true));
    s.async_pipeline = env_flag("AUTORUST_ASYNC", true);
    if (const char *m = getenv("AUTORUST_MATH")) {
        if (std::string(m) == "exact") {  // settings.rs:202-208: exact mode turns the matrix units off
            s.math_exact = true;
            s.tensor_cores = false;
        }
    }
    return s;
}

// ---- device ---------------------------------------------------------------------------

void Device::check(int rc) const
{
    if (rc != ARHIP_OK) throw std::runtime_error(std::string("TGERR: arhip ") + std::to_string(rc) + ": " + arhip_last_error());
}

Device::Device(int ordinal) : ordinal_(ordinal)
{
    const int rc = arhip_open(ordinal, &dev_);
    if (rc != ARHIP_OK) throw std::runtime_error(std::string("TGERR: arhip ") + std::to_string(rc) + ": " + arhip_last_error());
}

Device::~Device()
{
    for (auto &kv : free_)
        for (void *p : kv.second) arhip_free(dev_, p);
    arhip_close(dev_);
}

void *Device::alloc(size_t bytes)
{
    if (bytes == 0) return nullptr;
    auto it = free_.find(bytes);
    if (it != free_.end() && !it->second.empty()) {
        void *p = it->second.back();
        it->second.pop_back();
        return p;
    }
    void *p = nullptr;
    check(arhip_alloc(dev_, bytes, &p));
    ++raw_allocs_;
    return p;
}

void Device::release(void *p, size_t bytes)
{
    if (!p) return;
    auto &v = free_[bytes];
    if (v.size() < 32) {  // device.rs:128-203: at most 32 cached blocks per size
        v.push_back(p);
    } else {
        arhip_free(dev_, p);
    }
}

Storage::~Storage()
{
    if (dev && ptr) dev->release(ptr, bytes);
}

// ---- tensors --------------------------------------------------------------------------

static size_t esize(DType d) { return d == DType::BFloat16 ? 2 : 4; }

int64_t Tensor::numel() const
{
    int64_t n = 1;
    for (auto s : shape_) n *= s;
    return n;
}

Tensor Tensor::empty(const std::shared_ptr<Device> &dev, const std::vector<int64_t> &shape, DType dtype)
{
    Tensor t;
    t.shape_ = shape;
    t.dtype_ = dtype;
    t.st_ = std::make_shared<Storage>();
    t.st_->dev = dev;
    t.st_->bytes = (size_t)t.numel() * esize(dtype);
    t.st_->ptr = dev->alloc(t.st_->bytes);
    return t;
}

Tensor Tensor::from_slice(const std::shared_ptr<Device> &dev, const float *data, const std::vector<int64_t> &shape, DType dtype)
{
    if (dtype == DType::Other) throw std::runtime_error("TGERR: from_slice: only f32 and bf16 tensors exist on this device");
    Tensor t = empty(dev, shape, dtype);
    const int64_t n = t.numel();
    if (n == 0) return t;
    if (dtype == DType::Float32) {
        dev->check(arhip_copyin(dev->handle(), t.ptr(), data, (size_t)n * 4));
    } else {
        // cast on the device (round to nearest even, dtype/mod.rs:973-981) through an f32 staging buffer
        void *tmp = dev->alloc((size_t)n * 4);
        dev->check(arhip_copyin(dev->handle(), tmp, data, (size_t)n * 4));
        dev->check(arhip_cast_bf16(dev->handle(), (const float *)tmp, (uint16_t *)t.ptr(), n, 1, nullptr));
        dev->release(tmp, (size_t)n * 4);
    }
    return t;
}

Tensor Tensor::reshape(const std::vector<int64_t> &shape) const
{
    int64_t n = 1;
    for (auto s : shape) n *= s;
    if (n != numel()) throw std::runtime_error("TGERR: reshape: element count differs");
    Tensor t = *this;
    t.shape_ = shape;
    return t;
}

std::vector<float> Tensor::to_list() const
{
    const int64_t n = numel();
    std::vector<float> out((size_t)n);
    if (n == 0) return out;
    auto &dev = st_->dev;
    if (dtype_ == DType::Float32) {
        dev->check(arhip_copyout(dev->handle(), out.data(), ptr(), (size_t)n * 4));
    } else {
        std::vector<uint16_t> raw((size_t)n);
        dev->check(arhip_copyout(dev->handle(), raw.data(), ptr(), (size_t)n * 2));
        for (int64_t i = 0; i < n; ++i) {
            const uint32_t bits = (uint32_t)raw[(size_t)i] << 16;
            std::memcpy(&out[(size_t)i], &bits, 4);
        }
    }
    return out;
}

// ---- dispatcher -----------------------------------------------------------------------

static void note_once(std::once_flag &flag, const char *msg)
{
    std::call_once(flag, [msg] { std::fprintf(stderr, "%s\n", msg); });
}

Kernel plan_fused(const std::vector<int64_t> &q, const std::vector<int64_t> &k, const std::vector<int64_t> &v,
                  DType qd, DType kd, DType vd, const std::vector<int64_t> *mask_shape, DType mask_dtype,
                  bool enable_gqa, bool quantized, const Settings &st, bool *sage_declined)
{
    if (sage_declined) *sage_declined = false;
    if (q.size() != 4 || k.size() != 4 || v.size() != 4) return Kernel::None;            // :358-369
    const int64_t b = q[0], h = q[1], n = q[2], d = q[3];
    const int64_t hk = k[1], nk = k[2], dk = k[3], hv = v[1], nv = v[2], dv = v[3];
    if (k[0] != b || v[0] != b) return Kernel::None;
    if (nk != n || nv != n || dk != d || dv != d || hk != hv) return Kernel::None;       // :372-374
    if (enable_gqa) {
        if (hk <= 0 || h % hk != 0) return Kernel::None;                                 // :375-378
    } else if (hk != h) {
        return Kernel::None;                                                             // :379-381
    }
    if (qd != DType::Float32 && qd != DType::BFloat16) return Kernel::None;              // :382-385
    if (kd != qd || vd != qd) return Kernel::None;                                       // :386-388
    if (mask_shape) {  // dense additive f32 [n, n] only (:391-396)
        if (mask_dtype != DType::Float32 || mask_shape->size() != 2 || (*mask_shape)[0] != n || (*mask_shape)[1] != n)
            return Kernel::None;
    }
    const int dt = qd == DType::BFloat16 ? ARHIP_BF16 : ARHIP_F32;
    // Sage: the reference takes f32 tensors only (:411-414); bf16 tensors are accepted here too.
    const bool sage = quantized && st.tensor_cores && arhip_attn_supported(ARHIP_ATTN_SAGE, n, d, dt);
    if (quantized && !sage && sage_declined) *sage_declined = true;                      // :420-422
    if (sage) return Kernel::Sage;
    if (!arhip_attn_supported(ARHIP_ATTN_FLASH, n, d, dt)) return Kernel::None;
    if (qd == DType::BFloat16) return st.tensor_cores ? Kernel::FlashBf16 : Kernel::None;  // :427-429, bf16 needs the matrix units
    // f32 tensors: the reference prefers its TF32 kernel; CDNA4 has no such MFMA, so f32 runs exact
    return Kernel::FlashF32;                                                             // :451
}

bool wants_fused(std::optional<AttentionKind> force, const Settings &st, double dropout_p, bool has_session, bool *quantized)
{
    const AttentionKind requested = force.value_or(st.attention);     // explicit calls are never overridden
    if (quantized) *quantized = requested == AttentionKind::Sage;
    return effective(requested) != AttentionKind::Sdpa && dropout_p == 0.0 && has_session;
}

uint64_t selections(Kernel k) { return k == Kernel::None ? 0 : arhip_selections((int)k); }

std::optional<Tensor> fused_attention(const Tensor &q, const Tensor &k, const Tensor &v, Session &sess, const Settings &st)
{
    return fused_attention_ex(q, k, v, nullptr, false, false, false, sess, st);
}

std::optional<Tensor> fused_attention_kind(const Tensor &q, const Tensor &k, const Tensor &v, AttentionKind kind,
                                           Session &sess, const Settings &st)
{
    return fused_attention_ex(q, k, v, nullptr, false, false, kind == AttentionKind::Sage, sess, st);
}

std::optional<Tensor> fused_attention_ex(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *attn_mask,
                                         bool is_causal, bool enable_gqa, bool quantized, Session &sess, const Settings &st)
{
    static std::once_flag sage_note;
    bool sage_declined = false;
    std::vector<int64_t> mshape;
    if (attn_mask) mshape = attn_mask->shape();
    const Kernel kern = plan_fused(q.shape(), k.shape(), v.shape(), q.dtype(), k.dtype(), v.dtype(),
                                   attn_mask ? &mshape : nullptr, attn_mask ? attn_mask->dtype() : DType::Float32,
                                   enable_gqa, quantized, st, &sage_declined);
    if (sage_declined)
        note_once(sage_note, "[attention] sage: quantized attention is not available for this shape/settings: using the exact kernel");
    if (kern == Kernel::None) return std::nullopt;

    const int64_t b = q.shape()[0], h = q.shape()[1], n = q.shape()[2], d = q.shape()[3], hk = k.shape()[1];
    auto dev = q.device();
    const float scale = 1.0f / std::sqrt((float)d);
    // out: bf16 for bf16 tensors, f32 otherwise (:514-530); no host-side zero fill is needed,
    // the kernels write every element
    Tensor out = Tensor::empty(dev, {b, h, n, d}, q.dtype());
    const Tensor mask = attn_mask ? *attn_mask : Tensor();

    HostCall call;
    call.device = dev->name();
    call.global[0] = (n + 63) / 64;  // what the reference's launch would use (BQ = 64)
    call.global[1] = b * h;
    call.global[2] = 1;
    call.vals = {n, d, (int64_t)is_causal, (int64_t)(attn_mask != nullptr), h, hk};
    call.bufs = {q, k, v, out};
    if (attn_mask) call.bufs.push_back(mask);
    const float *mptr = attn_mask ? (const float *)mask.ptr() : nullptr;

    if (kern == Kernel::Sage) {
        call.name = "ar_flash_sage";
        const int in_dt = q.dtype() == DType::BFloat16 ? ARHIP_BF16 : ARHIP_F32;
        const int64_t bq = st.sage_block_q, bk = st.sage_block_k;
        const bool smooth = st.sage_smooth_k;
        call.run = [=]() {
            arhip_device *hd = dev->handle();
            const int64_t nq = b * h * n * d, nkv = b * hk * n * d;
            const int64_t nqb = (n + bq - 1) / bq, nkb = (n + bk - 1) / bk;
            // scratch from the free-list allocator: repeated calls do not reach hipMalloc
            const size_t ws_bytes = arhip_sage_quant_workspace(b, hk, n, d);
            void *q8 = dev->alloc((size_t)nq), *k8 = dev->alloc((size_t)nkv);
            void *sq = dev->alloc((size_t)(b * h * nqb) * 4), *sk = dev->alloc((size_t)(b * hk * nkb) * 4);
            void *mean = dev->alloc((size_t)(b * hk * d) * 4), *ws = dev->alloc(ws_bytes);
            void *vb = in_dt == ARHIP_F32 ? dev->alloc((size_t)nkv * 2) : nullptr;
            dev->check(arhip_sage_quant(hd, q.ptr(), (int8_t *)q8, (float *)sq, nullptr, nullptr, b, h, n, d, bq, in_dt, 0, 0, nullptr));
            dev->check(arhip_sage_quant(hd, k.ptr(), (int8_t *)k8, (float *)sk, (float *)mean, ws, b, hk, n, d, bk, in_dt,
                                        smooth ? 1 : 0, 0, nullptr));
            const uint16_t *vptr = (const uint16_t *)v.ptr();
            if (vb) {
                dev->check(arhip_cast_bf16(hd, (const float *)v.ptr(), (uint16_t *)vb, nkv, 0, nullptr));
                vptr = (const uint16_t *)vb;
            }
            dev->check(arhip_sage_fwd(hd, (const int8_t *)q8, (const int8_t *)k8, (const float *)sq, (const float *)sk, vptr,
                                      out.ptr(), mptr, nullptr, b, h, hk, n, d, bq, bk, is_causal, in_dt, scale, nullptr,
                                      nullptr, 1, nullptr));
            dev->release(q8, (size_t)nq); dev->release(k8, (size_t)nkv);
            dev->release(sq, (size_t)(b * h * nqb) * 4); dev->release(sk, (size_t)(b * hk * nkb) * 4);
            dev->release(mean, (size_t)(b * hk * d) * 4); dev->release(ws, ws_bytes);
            if (vb) dev->release(vb, (size_t)nkv * 2);
        };
    } else {
        const int dt = kern == Kernel::FlashBf16 ? ARHIP_BF16 : ARHIP_F32;
        call.name = kern == Kernel::FlashBf16 ? "ar_flash_bf16" : "ar_flash_f32";
        call.run = [=]() {
            dev->check(arhip_flash_fwd(dev->handle(), q.ptr(), k.ptr(), v.ptr(), out.ptr(), mptr, nullptr, b, h, hk, n, d,
                                       is_causal, dt, scale, 1, nullptr));
        };
    }
    // Record the launch for replay and run it now (flash_attention.rs:696-701).
    sess.capture_host(call);
    call.exec();
    return out;
}

// ---- Tensor API -----------------------------------------------------------------------

Tensor Tensor::attention_kind(const Tensor &key, const Tensor &value, const Tensor *mask, double dropout_p, bool is_causal,
                              std::optional<AttentionKind> force, Session *sess, const Settings &st) const
{
    bool quantized = false;
    const bool fused = wants_fused(force, st, dropout_p, sess != nullptr, &quantized);
    // fewer K/V heads than Q heads means GQA (tensor/mod.rs:2185-2195)
    const bool gqa = shape_.size() == 4 && key.shape().size() == 4 && key.shape()[1] != shape_[1];
    if (fused) {
        auto t = fused_attention_ex(*this, key, value, mask, is_causal, gqa, quantized, *sess, st);
        if (t) return *t;
    }
    // tensor/mod.rs:2207: the general scaled_dot_product_attention (generated kernels) runs here in the
    // reference; it is not part of this build, so the fallback is reported instead of being faked
    throw std::runtime_error("TGERR: attention: the fused kernels declined (shape, dtype, mask, dropout or no session); "
                             "the general SDPA path is the caller's");
}

Tensor Tensor::attention(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal) const
{
    return attention_kind(k, v, mask, dropout_p, is_causal, std::nullopt, nullptr, Settings());
}
Tensor Tensor::attention_with(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                              Session &sess, const Settings &st) const
{
    return attention_kind(k, v, mask, dropout_p, is_causal, std::nullopt, &sess, st);
}
Tensor Tensor::flash_attention_with(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                                    Session &sess, const Settings &st) const
{
    return attention_kind(k, v, mask, dropout_p, is_causal, AttentionKind::Flash, &sess, st);
}
Tensor Tensor::sage_attention_with(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                                   Session &sess, const Settings &st) const
{
    return attention_kind(k, v, mask, dropout_p, is_causal, AttentionKind::Sage, &sess, st);
}

}  // namespace autorust
