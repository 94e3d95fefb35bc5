// Test shim: a flat C view of the C++ host layer (autorust_host.h) so that the Python tests can
// drive Tensor / Session / fused_attention_ex the way the reference's Rust tests drive theirs.
// It is not part of the drop-in boundary (that is include/arhip.h).
#include <cstring>

#include "autorust_host.h"

using namespace autorust;

static thread_local std::string g_err;

struct arh_settings {
    int attention, tensor_cores, async_pipeline, math_exact;
    int64_t sage_block_q, sage_block_k;
    int sage_smooth_k;
    int sage_fp8;
};

static Settings to_settings(const arh_settings *s)
{
    Settings st;
    if (!s) return st;
    st.attention = (AttentionKind)s->attention;
    st.tensor_cores = s->tensor_cores != 0;
    st.async_pipeline = s->async_pipeline != 0;
    st.math_exact = s->math_exact != 0;
    st.sage_block_q = s->sage_block_q;
    st.sage_block_k = s->sage_block_k;
    st.sage_smooth_k = s->sage_smooth_k != 0;
    st.sage_fp8 = s->sage_fp8 != 0;
    return st;
}

struct SessionBox {
    Session sess;
    std::vector<HostCall> steps;
};

template <typename F>
static auto guard(F f, decltype(f()) fail) -> decltype(f())
{
    try {
        return f();
    } catch (const std::exception &e) {
        g_err = e.what();
        return fail;
    }
}

extern "C" {

const char *arh_last_error(void) { return g_err.c_str(); }

void arh_settings_default(arh_settings *out)
{
    const Settings s;
    *out = {(int)s.attention, s.tensor_cores, s.async_pipeline, s.math_exact, s.sage_block_q, s.sage_block_k, s.sage_smooth_k, s.sage_fp8};
}
void arh_settings_from_env(arh_settings *out)
{
    const Settings s = Settings::from_env();
    *out = {(int)s.attention, s.tensor_cores, s.async_pipeline, s.math_exact, s.sage_block_q, s.sage_block_k, s.sage_smooth_k, s.sage_fp8};
}
const char *arh_attention_kind_name(int k) { return name((AttentionKind)k); }
int arh_attention_kind_from_str(const char *s) { return (int)attention_kind_from_str(s); }

void *arh_device_open(int ordinal)
{
    return guard([&]() -> void * { return new std::shared_ptr<Device>(std::make_shared<Device>(ordinal)); }, nullptr);
}
void arh_device_close(void *d) { delete (std::shared_ptr<Device> *)d; }
uint64_t arh_device_raw_allocs(void *d) { return (*(std::shared_ptr<Device> *)d)->raw_allocs(); }
int arh_device_name(void *d, char *out, int cap)
{
    const std::string n = (*(std::shared_ptr<Device> *)d)->name();
    std::strncpy(out, n.c_str(), (size_t)cap);
    return (int)n.size();
}

void *arh_tensor_from_slice(void *d, const float *data, const int64_t *shape, int ndim, int dtype)
{
    return guard([&]() -> void * {
        std::vector<int64_t> shp(shape, shape + ndim);
        return new Tensor(Tensor::from_slice(*(std::shared_ptr<Device> *)d, data, shp, (DType)dtype));
    }, nullptr);
}
void *arh_tensor_from_i32(void *d, const int32_t *data, const int64_t *shape, int ndim)
{
    return guard([&]() -> void * {
        std::vector<int64_t> shp(shape, shape + ndim);
        return new Tensor(Tensor::from_i32(*(std::shared_ptr<Device> *)d, data, shp));
    }, nullptr);
}
void arh_tensor_free(void *t) { delete (Tensor *)t; }
int64_t arh_tensor_numel(void *t) { return ((Tensor *)t)->numel(); }
int arh_tensor_dtype(void *t) { return (int)((Tensor *)t)->dtype(); }
int arh_tensor_shape(void *t, int64_t *out, int cap)
{
    const auto &s = ((Tensor *)t)->shape();
    for (int i = 0; i < (int)s.size() && i < cap; ++i) out[i] = s[(size_t)i];
    return (int)s.size();
}
int arh_tensor_to_list(void *t, float *out)
{
    return guard([&]() -> int {
        const auto v = ((Tensor *)t)->to_list();
        std::memcpy(out, v.data(), v.size() * 4);
        return 0;
    }, -1);
}

void *arh_session_new(void) { return new SessionBox(); }
void arh_session_free(void *s) { delete (SessionBox *)s; }
void arh_session_begin_capture(void *s) { ((SessionBox *)s)->sess.begin_capture(); }
int arh_session_end_capture(void *s)
{
    auto *b = (SessionBox *)s;
    b->steps = b->sess.end_capture();
    return (int)b->steps.size();
}
int arh_session_step_info(void *s, int i, char *name, int cap, int64_t *global3, int64_t *vals6)
{
    auto *b = (SessionBox *)s;
    if (i < 0 || i >= (int)b->steps.size()) return -1;
    const HostCall &c = b->steps[(size_t)i];
    std::strncpy(name, c.name.c_str(), (size_t)cap);
    for (int j = 0; j < 3; ++j) global3[j] = c.global[j];
    for (int j = 0; j < 6 && j < (int)c.vals.size(); ++j) vals6[j] = c.vals[(size_t)j];
    return 0;
}
// the rest of a captured launch: code object path, workgroup shape, number of buffers / scalars,
// and the (slot, dtype) signature as pairs
int arh_session_step_detail(void *s, int i, char *src, int cap, int64_t *local3, int *nbufs, int *nvals, int64_t *sig_pairs,
                            int sig_cap)
{
    auto *b = (SessionBox *)s;
    if (i < 0 || i >= (int)b->steps.size()) return -1;
    const HostCall &c = b->steps[(size_t)i];
    std::strncpy(src, c.src.c_str(), (size_t)cap);
    for (int j = 0; j < 3; ++j) local3[j] = c.local ? (*c.local)[(size_t)j] : -1;
    *nbufs = (int)c.bufs.size();
    *nvals = (int)c.vals.size();
    for (int j = 0; j < (int)c.signature.size() && 2 * j + 1 < sig_cap; ++j) {
        sig_pairs[2 * j] = c.signature[(size_t)j].first;
        sig_pairs[2 * j + 1] = (int64_t)c.signature[(size_t)j].second;
    }
    return (int)c.signature.size();
}
int arh_session_replay(void *s)
{
    return guard([&]() -> int {
        Session::replay(((SessionBox *)s)->steps);
        return 0;
    }, -1);
}

// api: 0 attention (no session), 1 attention_with, 2 flash_attention_with, 3 sage_attention_with
// key_lengths: an Int32 [b] tensor or NULL (the *_with entry points only)
void *arh_attention(void *q, void *k, void *v, void *mask, double dropout_p, int is_causal, int api, void *sess,
                    const arh_settings *st, void *key_lengths)
{
    return guard([&]() -> void * {
        const Tensor &tq = *(Tensor *)q, &tk = *(Tensor *)k, &tv = *(Tensor *)v;
        const Tensor *tm = (const Tensor *)mask, *tl = (const Tensor *)key_lengths;
        if (api == 0 && tl) throw std::runtime_error("TGERR: key lengths need a session (the *_with entry points)");
        const Settings s = to_settings(st);
        Session *ss = sess ? &((SessionBox *)sess)->sess : nullptr;
        if (api != 0 && !ss) throw std::runtime_error("TGERR: a session is required for the *_with entry points");
        switch (api) {
        case 0: return new Tensor(tq.attention(tk, tv, tm, dropout_p, is_causal != 0));
        case 1: return new Tensor(tq.attention_with(tk, tv, tm, dropout_p, is_causal != 0, *ss, s, tl));
        case 2: return new Tensor(tq.flash_attention_with(tk, tv, tm, dropout_p, is_causal != 0, *ss, s, tl));
        default: return new Tensor(tq.sage_attention_with(tk, tv, tm, dropout_p, is_causal != 0, *ss, s, tl));
        }
    }, nullptr);
}

// fused_attention (kind < 0) / fused_attention_kind: the thin wrappers of
// src/models/flash_attention.rs:292-320.  Returns NULL with an empty error when the kernels
// decline (the reference's None).
void *arh_fused_attention(void *q, void *k, void *v, int kind, void *sess, const arh_settings *st)
{
    g_err.clear();
    return guard([&]() -> void * {
        const Tensor &tq = *(Tensor *)q, &tk = *(Tensor *)k, &tv = *(Tensor *)v;
        Session &ss = ((SessionBox *)sess)->sess;
        const Settings s = to_settings(st);
        std::optional<Tensor> r = kind < 0 ? fused_attention(tq, tk, tv, ss, s)
                                           : fused_attention_kind(tq, tk, tv, (AttentionKind)kind, ss, s);
        return r ? (void *)new Tensor(*r) : nullptr;
    }, nullptr);
}

// fused_attention_train / fused_attention_backward (src/models/flash_attention.rs:789-977).
// Return 1 and fill the outputs, 0 when the kernels decline (the reference's None), -1 on error.
int arh_fused_attention_train(void *q, void *k, void *v, void *mask, int is_causal, void *sess, void **out, void **lse)
{
    g_err.clear();
    return guard([&]() -> int {
        auto r = fused_attention_train(*(Tensor *)q, *(Tensor *)k, *(Tensor *)v, (const Tensor *)mask, is_causal != 0,
                                       ((SessionBox *)sess)->sess);
        if (!r) return 0;
        *out = new Tensor(r->out);
        *lse = new Tensor(r->lse);
        return 1;
    }, -1);
}

int arh_fused_attention_backward(void *q, void *k, void *v, void *out, void *lse, void *dout, void *mask, int is_causal,
                                 void *sess, void **dq, void **dk, void **dv)
{
    g_err.clear();
    return guard([&]() -> int {
        auto r = fused_attention_backward(*(Tensor *)q, *(Tensor *)k, *(Tensor *)v, *(Tensor *)out, *(Tensor *)lse,
                                          *(Tensor *)dout, (const Tensor *)mask, is_causal != 0, ((SessionBox *)sess)->sess);
        if (!r) return 0;
        *dq = new Tensor(r->dq);
        *dk = new Tensor(r->dk);
        *dv = new Tensor(r->dv);
        return 1;
    }, -1);
}

int arh_plan_fused(const int64_t *q, int qn, const int64_t *k, int kn, const int64_t *v, int vn, int qd, int kd, int vd,
                   const int64_t *mask, int mn, int mask_dtype, int enable_gqa, int quantized, const arh_settings *st,
                   int *sage_declined)
{
    std::vector<int64_t> qs(q, q + qn), ks(k, k + kn), vs(v, v + vn), ms;
    if (mask) ms.assign(mask, mask + mn);
    bool declined = false;
    const Kernel kern = plan_fused(qs, ks, vs, (DType)qd, (DType)kd, (DType)vd, mask ? &ms : nullptr, (DType)mask_dtype,
                                   enable_gqa != 0, quantized != 0, to_settings(st), &declined);
    if (sage_declined) *sage_declined = declined;
    return (int)kern;
}

int arh_wants_fused(int force, const arh_settings *st, double dropout_p, int has_session, int *quantized)
{
    bool qz = false;
    std::optional<AttentionKind> f;
    if (force >= 0) f = (AttentionKind)force;
    const bool w = wants_fused(f, to_settings(st), dropout_p, has_session != 0, &qz);
    if (quantized) *quantized = qz;
    return w;
}

// Device::run_host_kernel with device pointers and 32-bit scalars (the generic seam, for tests of
// its own behaviour: argument marshalling, the KPROF line).  Returns 0, or -1 with arh_last_error().
int arh_run_host_kernel(void *d, const char *src, const char *name, void **bufs, int nbufs, const int64_t *vals, int nvals,
                        const int64_t *global3, const int64_t *local3, int wait, double *secs)
{
    return guard([&]() -> int {
        std::vector<std::pair<int64_t, DType>> sig;
        for (int i = 0; i < nbufs; ++i) sig.emplace_back(i, DType::Float32);
        for (int i = 0; i < nvals; ++i) sig.emplace_back(nbufs + i, DType::Int32);
        const std::vector<void *> b(bufs, bufs + nbufs);
        const std::vector<int64_t> v(vals, vals + nvals);
        const std::array<int64_t, 3> loc = {local3[0], local3[1], local3[2]};
        const auto r = (*(std::shared_ptr<Device> *)d)->run_host_kernel(src, name, sig, b, global3, loc, v, wait != 0);
        if (secs) *secs = r ? *r : -1.0;
        return 0;
    }, -1);
}
void *arh_tensor_ptr(void *t) { return ((Tensor *)t)->ptr(); }

uint64_t arh_selections(int kernel) { return selections((Kernel)kernel); }

}  // extern "C"
