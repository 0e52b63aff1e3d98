// C++ host adapter over the C ABI (include/tritium_mi355x.h): the backend-adapter interface of the
// reference, restated in C++ because the reference's host language (Rust) has no toolchain here.
// Names, argument meaning and error behaviour follow crates/tritium-spec/src/lib.rs:64-78 (MpGemm),
// :147-158 (DeviceBuffer), :166-333 (TernaryBackend), :382-405 (BackendError), caps.rs:7-67
// (DeviceCaps) and crates/tritium-runtime/src/lib.rs:73-217 (BackendEntry, Registry).
// Header-only; link with libtritium_mi355x.so.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <functional>
#include <memory>
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "../../include/tritium_mi355x.h"

namespace tritium {

enum class TernaryFormat { Tq1_0 = TK_FORMAT_TQ1_0, Tq2_0 = TK_FORMAT_TQ2_0, I2sInt8 = TK_FORMAT_I2S_INT8 };

struct GemmShape {
  size_t m, n, k;
  uint64_t macs() const { return (uint64_t)m * n * k; }
  bool buffers_fit(size_t act_len, size_t weight_len, size_t out_len) const {
    return act_len == m * k && weight_len == n * k && out_len == m * n;
  }
};

// BackendError: a value, never thrown by the backends themselves.
struct BackendError {
  enum Kind { ShapeMismatch = 1, UnsupportedFormat = 2, OutOfMemory = 3, InvalidInput = 4, Backend = 5 } kind;
  size_t expected = 0, got = 0;  // ShapeMismatch{expected,got}; OutOfMemory{requested = expected}
  std::string message;
  static BackendError shape(size_t e, size_t g) {
    return {ShapeMismatch, e, g, "shape mismatch: expected " + std::to_string(e) + ", got " + std::to_string(g)};
  }
  static BackendError from_status(int code) {
    BackendError e{(Kind)code, 0, 0, tk_last_error()};
    if (code == TK_ERR_SHAPE_MISMATCH || code == TK_ERR_OUT_OF_MEMORY) tk_last_mismatch(&e.expected, &e.got);
    return e;
  }
};
using Status = std::optional<BackendError>;  // nullopt == Ok(())

struct DeviceCaps {
  std::string backend, device_name;
  std::vector<std::string> features;
  uint64_t total_memory_bytes = 0;
  bool supports_imma = false, supports_fp8 = false;
  bool has_feature(const std::string &f) const {
    for (auto &x : features)
      if (x == f) return true;
    return false;
  }
};

class DeviceBuffer {
 public:
  virtual ~DeviceBuffer() = default;
  virtual size_t len_bytes() const = 0;
  bool is_empty() const { return len_bytes() == 0; }
};

struct MpGemm {
  const float *act;
  size_t act_len;
  const DeviceBuffer *weights;
  const float *scales;
  size_t scales_len;
  GemmShape shape;
  TernaryFormat format;
  float *out;
  size_t out_len;
};

// Operands of the VJP of one packed mpGEMM (crates/tritium-spec/src/lib.rs:93-117); grad_bias may be null.
struct MpGemmProjectedVjp {
  const float *act;
  size_t act_len;
  const DeviceBuffer *weights;
  const float *scales;
  size_t scales_len;
  const float *grad_output;
  size_t grad_output_len;
  GemmShape shape;
  TernaryFormat format;
  float *grad_act;
  size_t grad_act_len;
  float *grad_projected_weight;
  size_t grad_projected_weight_len;
  float *grad_bias;
  size_t grad_bias_len;
};

// Per-token int8 absmax quant of the trait's default fused path (crates/tritium-spec/src/lib.rs:351-378):
// one divide 127/gamma, one multiply, ties to even, clamp [-128,127]; a zero row gives zeros and scale 0.
inline void quantize_act_int8(const float *act, size_t m, size_t k, float *q, float *scale) {
  for (size_t r = 0; r < m; ++r) {
    const float *row = act + r * k;
    float gamma = 0.0f;
    for (size_t c = 0; c < k; ++c) {
      float a = std::fabs(row[c]);
      if (a > gamma) gamma = a;
    }
    if (gamma == 0.0f) {
      for (size_t c = 0; c < k; ++c) q[r * k + c] = 0.0f;
      scale[r] = 0.0f;
      continue;
    }
    volatile float s = 127.0f / gamma;
    for (size_t c = 0; c < k; ++c) {
      volatile float v = row[c] * s;
      float rr = std::nearbyint(v);
      q[r * k + c] = rr < -128.0f ? -128.0f : (rr > 127.0f ? 127.0f : rr);
    }
    scale[r] = gamma / 127.0f;
  }
}

class TernaryBackend {
 public:
  virtual ~TernaryBackend() = default;
  virtual const std::string &device_id() const = 0;
  virtual const std::string &physical_device_id() const { return device_id(); }
  virtual DeviceCaps capabilities() const = 0;
  virtual Status upload_weights(const uint8_t *packed, size_t len, GemmShape shape, TernaryFormat format,
                                std::unique_ptr<DeviceBuffer> *out) = 0;
  virtual Status mpgemm(const MpGemm &p) = 0;
  // inference-only default (crates/tritium-spec/src/lib.rs:221-226)
  virtual Status mpgemm_projected_vjp(const MpGemmProjectedVjp &) {
    return BackendError{BackendError::Backend, 0, 0, "backend `" + device_id() + "` does not implement packed mpGEMM VJP"};
  }
  // default: host quant -> mpgemm -> fold (crates/tritium-spec/src/lib.rs:266-318)
  virtual Status mpgemm_with_act_quant(const MpGemm &p) {
    const GemmShape s = p.shape;
    if (p.act_len != s.m * s.k) return BackendError::shape(s.m * s.k, p.act_len);
    if (p.out_len != s.m * s.n) return BackendError::shape(s.m * s.n, p.out_len);
    if (p.scales_len != s.n) return BackendError::shape(s.n, p.scales_len);
    std::vector<float> q(s.m * s.k), as(s.m);
    quantize_act_int8(p.act, s.m, s.k, q.data(), as.data());
    MpGemm inner = p;
    inner.act = q.data();
    if (Status e = mpgemm(inner)) return e;
    for (size_t r = 0; r < s.m; ++r)
      for (size_t c = 0; c < s.n; ++c) p.out[r * s.n + c] = p.out[r * s.n + c] * as[r];
    return std::nullopt;
  }
  virtual void *as_concrete() { return nullptr; }
};

// ---- the MI355X backend ---------------------------------------------------------------------

class Mi355xBuffer : public DeviceBuffer {
 public:
  explicit Mi355xBuffer(tk_weights *h) : h_(h) {}
  ~Mi355xBuffer() override { tk_free_weights(h_); }  // owns device memory, frees on drop
  size_t len_bytes() const override { return tk_weights_len_bytes(h_); }
  tk_weights *handle() const { return h_; }

 private:
  tk_weights *h_;
};

class Mi355xBackend : public TernaryBackend {
 public:
  // RocmBackend::new(ordinal) (crates/tritium-rocm/src/rocm.rs:234-300): an Err, never a panic, without a device
  static Status create(int ordinal, std::unique_ptr<Mi355xBackend> *out) {
    tk_ctx *ctx = nullptr;
    if (int rc = tk_init(ordinal, &ctx)) return BackendError::from_status(rc);
    out->reset(new Mi355xBackend(ctx));
    return std::nullopt;
  }
  ~Mi355xBackend() override { tk_destroy(ctx_); }
  const std::string &device_id() const override { return id_; }
  DeviceCaps capabilities() const override {
    tk_device_info info{};
    tk_device_info_get(ctx_, &info);
    DeviceCaps c;
    c.backend = "mi355x";
    c.device_name = info.name;
    c.features = {"hip", "gfx950", "tq2_0", "tq1_0", "mfma_i8", "act_quant_i8", "additive_planes", "rmsnorm_quant_i8", "salt_block_scales"};
    c.total_memory_bytes = info.total_memory_bytes;
    c.supports_imma = true;
    return c;
  }
  Status upload_weights(const uint8_t *packed, size_t len, GemmShape shape, TernaryFormat format,
                        std::unique_ptr<DeviceBuffer> *out) override {
    tk_weights *w = nullptr;
    if (int rc = tk_upload_weights(ctx_, packed, len, shape.n, shape.k, (int)format, &w))
      return BackendError::from_status(rc);
    out->reset(new Mi355xBuffer(w));
    return std::nullopt;
  }
  Status mpgemm(const MpGemm &p) override { return call(tk_mpgemm, p); }
  Status mpgemm_with_act_quant(const MpGemm &p) override { return call(tk_mpgemm_with_act_quant, p); }
  Status mpgemm_projected_vjp(const MpGemmProjectedVjp &p) override {
    auto *buf = dynamic_cast<const Mi355xBuffer *>(p.weights);
    if (!buf) return BackendError{BackendError::InvalidInput, 0, 0, "buffer is not a Mi355xBuffer"};
    if (int rc = tk_mpgemm_projected_vjp(ctx_, p.act, p.act_len, buf->handle(), p.scales, p.scales_len, p.grad_output,
                                         p.grad_output_len, p.shape.m, p.shape.n, p.shape.k, (int)p.format, p.grad_act,
                                         p.grad_act_len, p.grad_projected_weight, p.grad_projected_weight_len,
                                         p.grad_bias, p.grad_bias_len))
      return BackendError::from_status(rc);
    return std::nullopt;
  }
  void *as_concrete() override { return this; }
  tk_ctx *ctx() const { return ctx_; }  // the device-resident extension is the C ABI itself

 private:
  explicit Mi355xBackend(tk_ctx *ctx) : ctx_(ctx), id_(tk_device_id(ctx)) {}
  template <typename F>
  Status call(F fn, const MpGemm &p) {
    auto *buf = dynamic_cast<const Mi355xBuffer *>(p.weights);
    if (!buf) return BackendError{BackendError::InvalidInput, 0, 0, "buffer is not a Mi355xBuffer"};
    if (int rc = fn(ctx_, p.act, p.act_len, buf->handle(), p.scales, p.scales_len, p.shape.m, p.shape.n, p.shape.k,
                    (int)p.format, p.out, p.out_len))
      return BackendError::from_status(rc);
    return std::nullopt;
  }
  tk_ctx *ctx_;
  std::string id_;
};

// ---- registration -----------------------------------------------------------------------------

struct BackendEntry {
  std::string name;
  std::function<Status(std::unique_ptr<TernaryBackend> *)> init;
};

inline std::vector<BackendEntry> &backends() {
  static std::vector<BackendEntry> v = {{"mi355x", [](std::unique_ptr<TernaryBackend> *out) -> Status {
                                           std::unique_ptr<Mi355xBackend> b;
                                           if (Status e = Mi355xBackend::create(0, &b)) return e;
                                           *out = std::move(b);
                                           return std::nullopt;
                                         }}};
  return v;
}

// A failing init is written to stderr and skipped; an empty registry is a valid result.
class Registry {
 public:
  explicit Registry(const std::vector<BackendEntry> &entries = backends()) {
    for (auto &e : entries) {
      std::unique_ptr<TernaryBackend> b;
      if (Status err = e.init(&b)) {
        std::fprintf(stderr, "tritium-runtime: backend `%s` failed to initialise, skipping: %s\n", e.name.c_str(),
                     err->message.c_str());
        continue;
      }
      items_.emplace_back(e.name, std::move(b));
    }
  }
  TernaryBackend *get(const std::string &name) const {
    for (auto &it : items_)
      if (it.first == name) return it.second.get();
    return nullptr;
  }
  std::vector<DeviceCaps> enumerate() const {
    std::vector<DeviceCaps> v;
    for (auto &it : items_) v.push_back(it.second->capabilities());
    return v;
  }
  size_t len() const { return items_.size(); }
  bool is_empty() const { return items_.empty(); }

 private:
  std::vector<std::pair<std::string, std::unique_ptr<TernaryBackend>>> items_;
};

}  // namespace tritium
