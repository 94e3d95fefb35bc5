// C++ mirror of the reference's attention interface, above the libarhip C ABI.
//
// The reference is Rust; its toolchain is not available to this build, so the host side
// of the path is restated in C++ with the reference's names, argument meaning and error
// behaviour:
//   Tensor::{attention, attention_with, flash_attention[_with], sage_attention[_with]}
//                                               src/tensor/mod.rs:2045-2161
//   Tensor::attention_kind (policy)             src/tensor/mod.rs:2165-2208
//   fused_attention / fused_attention_kind / fused_attention_ex
//                                               src/models/flash_attention.rs:292-702
//   AttentionKind                               src/models/flash_attention.rs:709-747
//   Settings (attention, tensor_cores, math)    src/settings.rs:82-143, 202-232
//   Session::capture_host, HostCall::exec, Jit replay
//                                               src/engine/session.rs:138-146, 210-256; jit.rs:186-195
//   LruAllocator                                src/runtime/device.rs:128-203
// Errors are `throw std::runtime_error("TGERR: ...")`, the counterpart of the reference's
// `panic!("TGERR: ...")`.  A capability gap is never an error: fused_attention_ex returns
// std::nullopt and the caller takes its general (SDPA) path, which is outside this build.
#pragma once

#include <array>
#include <cstdint>
#include <map>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../../include/arhip.h"

namespace autorust {

enum class AttentionKind { Sdpa = 0, Flash = 1, Sage = 2 };
const char *name(AttentionKind k);                       // flash_attention.rs:731-737
inline AttentionKind effective(AttentionKind k) { return k; }  // flash_attention.rs:744-746
AttentionKind attention_kind_from_str(const std::string &s);   // settings.rs:209-213

// Other: anything else a tensor could be; Int8/Int32/Int64 only type scratch buffers and kernel scalars
enum class DType { Float32 = 0, BFloat16 = 1, Other = 2, Int8 = 3, Int32 = 4, Int64 = 5 };

struct Settings {
    AttentionKind attention = AttentionKind::Flash;  // AUTORUST_ATTN (default flash)
    bool tensor_cores = true;                        // AUTORUST_TENSOR_CORES / AUTORUST_TC
    bool async_pipeline = true;                      // AUTORUST_ASYNC (no effect on this device)
    bool math_exact = false;                         // AUTORUST_MATH=exact => tensor_cores = false
    // Sage extension of this build (the reference quantises per row and does not smooth K)
    int64_t sage_block_q = 128, sage_block_k = 64;
    bool sage_smooth_k = true;
    // `cuda_flash_sage::Options::fp8` (cuda_flash_sage.rs:53-54): E4M3 codes and the FP8 matrix instruction
    // instead of int8.  The reference switches it on wherever the device has FP8 tensor cores; here it
    // is opt-in (AUTORUST_SAGE_FP8=1) because the int8 path is the measured one.
    bool sage_fp8 = false;
    static Settings from_env();                      // settings.rs:174-282
};

// ---- device with the reference's free-list allocator --------------------------------
class Device {
public:
    explicit Device(int ordinal);
    ~Device();
    Device(const Device &) = delete;
    arhip_device *handle() const { return dev_; }
    std::string name() const { return ordinal_ == 0 ? "HIP" : "HIP:" + std::to_string(ordinal_); }
    int compute_units() const;
    void *alloc(size_t bytes);   // reuses a cached block of the same size (<= 32 kept per size)
    void release(void *p, size_t bytes);
    uint64_t raw_allocs() const { return raw_allocs_; }
    void check(int rc) const;    // throws "TGERR: ..." on failure
    // `Compiled::run_host_kernel` (src/runtime/device.rs:383-402) + `Prog::call`
    // (src/runtime/ops_cuda.rs:930-1019): `src` names the code object (a file path; loaded once and
    // cached like compile_cached does), arguments follow `signature`: slot < bufs.size() is that
    // buffer's device pointer, any other slot is vals[slot - bufs.size()] narrowed to the width of
    // its dtype.  global is the grid in workgroups, local the workgroup shape.  Returns the elapsed
    // device seconds when wait is set.
    std::optional<double> run_host_kernel(const std::string &src, const std::string &name,
                                          const std::vector<std::pair<int64_t, DType>> &signature,
                                          const std::vector<void *> &bufs, const int64_t global[3],
                                          const std::optional<std::array<int64_t, 3>> &local,
                                          const std::vector<int64_t> &vals, bool wait);
private:
    arhip_device *dev_ = nullptr;
    int ordinal_;
    std::map<size_t, std::vector<void *>> free_;
    std::map<std::string, void *> modules_;  // code object path -> loaded module
    std::map<std::string, uint64_t> module_keys_;  // code object path -> content hash (the key KPROF prints)
    uint64_t raw_allocs_ = 0;
};

// Path of the code object with the named attention kernels (autorust_amd/attn_kernels.hsaco):
// $AUTORUST_HIP_KERNELS, else the file next to this library.
std::string attention_kernels_src();

struct Storage {  // OpaqueT: base pointer + size, views share it (buffer.rs:32-39)
    std::shared_ptr<Device> dev;
    void *ptr = nullptr;
    size_t bytes = 0;
    ~Storage();
};

class Session;

class Tensor {
public:
    Tensor() = default;
    static Tensor from_slice(const std::shared_ptr<Device> &dev, const float *data, const std::vector<int64_t> &shape,
                             DType dtype);                       // tensor/mod.rs:1088
    static Tensor empty(const std::shared_ptr<Device> &dev, const std::vector<int64_t> &shape, DType dtype);
    // an Int32 tensor (the only integer tensors of this path: per-batch key lengths)
    static Tensor from_i32(const std::shared_ptr<Device> &dev, const int32_t *data, const std::vector<int64_t> &shape);
    size_t nbytes() const;
    Tensor reshape(const std::vector<int64_t> &shape) const;     // view: shares storage
    std::vector<float> to_list() const;                          // tensor/mod.rs:695 (bf16 widened to f32)
    const std::vector<int64_t> &shape() const { return shape_; }
    DType dtype() const { return dtype_; }
    int64_t numel() const;
    void *ptr() const { return st_ ? st_->ptr : nullptr; }
    const std::shared_ptr<Device> &device() const { return st_->dev; }
    bool defined() const { return (bool)st_; }

    // The public attention entry points (tensor/mod.rs:2045-2161).  When the policy or the kernels
    // decline, the call throws "TGERR: ... general SDPA path ..." because that path is outside this build.
    // `key_lengths` (optional, Int32 [b]) is a key-padding mask: batch i attends to keys [0, key_lengths[i])
    // only.  The reference reaches such masks through its general path (a broadcast bool mask,
    // tensor/mod.rs:2405-2447); here they stay on the fused kernels (the `*_lens` entry points).
    Tensor attention(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal) const;
    Tensor attention_with(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                          Session &sess, const Settings &st, const Tensor *key_lengths = nullptr) const;
    Tensor flash_attention_with(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                                Session &sess, const Settings &st, const Tensor *key_lengths = nullptr) const;
    Tensor sage_attention_with(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                               Session &sess, const Settings &st, const Tensor *key_lengths = nullptr) const;
private:
    Tensor attention_kind(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                          std::optional<AttentionKind> force, Session *sess, const Settings &st,
                          const Tensor *key_lengths) const;
    std::shared_ptr<Storage> st_;
    std::vector<int64_t> shape_;
    DType dtype_ = DType::Float32;
    friend std::optional<Tensor> fused_attention_ex(const Tensor &, const Tensor &, const Tensor &, const Tensor *, bool,
                                                    bool, bool, Session &, const Settings &, const Tensor *);
};

// ---- captured launches ----------------------------------------------------------------
struct HostCall {              // session.rs:210-256, field for field
    std::string device;        // "HIP"
    std::string src;           // the kernel "source": here the path of the gfx950 code object
    std::string name;          // entry point ("ar_flash_f32", "ar_flash_bf16", "ar_flash_sage", ...)
    std::vector<std::pair<int64_t, DType>> signature;  // (slot, dtype) argument list
    std::vector<Tensor> bufs;  // buffers in slot order, held so that a replay can resolve them
    int64_t global[3];         // launch grid
    std::optional<std::array<int64_t, 3>> local;       // launch block
    std::vector<int64_t> vals; // scalar arguments
    void exec() const;         // run_host_kernel(..., wait = true), session.rs:230-255
};

class Session {                // session.rs:44-193 (the part the path touches)
public:
    void begin_capture() { capturing_ = true; captured_.clear(); }
    std::vector<HostCall> end_capture() { capturing_ = false; return captured_; }
    void capture_host(const HostCall &c) { if (capturing_) captured_.push_back(c); }   // session.rs:138-146
    static void replay(const std::vector<HostCall> &steps) { for (auto &s : steps) s.exec(); }  // jit.rs:186-195
private:
    bool capturing_ = false;
    std::vector<HostCall> captured_;
};

// ---- dispatcher -----------------------------------------------------------------------
enum class Kernel { None = -1, FlashF32 = ARHIP_K_FLASH_F32, FlashBf16 = ARHIP_K_FLASH_BF16, Sage = ARHIP_K_SAGE };

// The launches one fused attention call consists of, in order (the pre-pass of the quantised
// path first, the attention kernel last), without running them: the `host_call` builders of
// src/runtime/cuda_flash{,_bf16,_sage}.rs (cuda_flash_bf16.rs:580-599).
// With `key_lengths` (Int32 [b]) the attention kernel is the `*_lens` twin and the lengths ride as one more
// buffer after the mask slot.
std::vector<HostCall> attention_host_calls(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *attn_mask,
                                           const Tensor &out, bool is_causal, Kernel kern, const Settings &st,
                                           const Tensor *key_lengths = nullptr);

// The gates of fused_attention_ex without touching a device (flash_attention.rs:358-472):
// which kernel would run, or Kernel::None (=> the caller's SDPA).
Kernel plan_fused(const std::vector<int64_t> &q, const std::vector<int64_t> &k, const std::vector<int64_t> &v,
                  DType qd, DType kd, DType vd, const std::vector<int64_t> *mask_shape, DType mask_dtype,
                  bool enable_gqa, bool quantized, const Settings &st, bool *sage_declined = nullptr);

// The policy of Tensor::attention_kind (tensor/mod.rs:2165-2208): fused iff kind != Sdpa and
// dropout_p == 0 and a session is given.
bool wants_fused(std::optional<AttentionKind> force, const Settings &st, double dropout_p, bool has_session,
                 bool *quantized);

std::optional<Tensor> fused_attention(const Tensor &q, const Tensor &k, const Tensor &v, Session &sess,
                                      const Settings &st);                                   // :292-299
std::optional<Tensor> fused_attention_kind(const Tensor &q, const Tensor &k, const Tensor &v, AttentionKind kind,
                                           Session &sess, const Settings &st);               // :303-320
std::optional<Tensor> fused_attention_ex(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *attn_mask,
                                         bool is_causal, bool enable_gqa, bool quantized, Session &sess,
                                         const Settings &st, const Tensor *key_lengths = nullptr);  // :348-702
uint64_t selections(Kernel k);   // cuda_flash_bf16.rs:458-461

// ---- training: forward with the saved log-sum-exp, and the backward ------------------------
// `fused_attention_train` / `fused_attention_backward` (src/models/flash_attention.rs:789-977):
// f32 only, 4-D, mask f32 [n, n] or none; anything else => std::nullopt (the caller keeps its
// graph path).  train returns (out [b,h,n,d], lse [b*h, n]); backward returns (dq, dk, dv).
struct TrainOut { Tensor out, lse; };
struct Grads { Tensor dq, dk, dv; };
std::optional<TrainOut> fused_attention_train(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *attn_mask,
                                              bool is_causal, Session &sess);
std::optional<Grads> fused_attention_backward(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor &out,
                                              const Tensor &lse, const Tensor &dout, const Tensor *attn_mask,
                                              bool is_causal, Session &sess);

}  // namespace autorust
