// tract_rocm.hpp — C++17 host-side mirror of tract's KV-cache operators over the C ABI of
// tract_rocm.h.  Header-only; names, argument meaning and error behaviour follow the reference
// operators (the same mirror exists in Python, tract_amd/ops.py):
//   InPlaceKvCache            transformers/src/ops/inplace_kv_cache.rs:28-114
//   InPlaceKvSdpa / State     transformers/src/ops/inplace_kv_cache.rs:131-290
//   Sdpa                      transformers/src/ops/sdpa.rs:83-89, 296-356
//   runtime_for_name          core/src/runtime.rs:223-250
//   QuantizedDynKeyValueCache / State   transformers/src/ops/quant_dyn_kv_cache.rs:283-495
//   QuantizedKvSdpa / State             transformers/src/ops/kv_quant.rs:242-355
// Every failing ABI call becomes a trocm::Error carrying the library's message, the way a
// TractResult Err carries its context.
#pragma once
#include <cmath>
#include <cstdint>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>
#include "tract_rocm.h"

namespace trocm {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};
inline void check(int rc) {
    if (rc != 0) throw Error(trocm_last_error());
}

enum class DatumType { F32 = TROCM_F32, F16 = TROCM_F16 };
inline size_t size_of(DatumType dt) { return dt == DatumType::F32 ? 4 : 2; }

class Runtime {
   public:
    std::string name() const { return "rocm"; }
    void check() const { trocm::check(trocm_device_sync()); }
};
inline Runtime runtime_for_name(const std::string &name, int device = 0) {
    if (name != "rocm") throw Error("Runtime \"" + name + "\" not found: only \"rocm\" is registered here");
    check(trocm_init(device));
    return Runtime();
}

// A dense device tensor (shape + datum type); move-only owner of its allocation.
class DeviceTensor {
   public:
    DeviceTensor() = default;
    DeviceTensor(std::vector<int64_t> shape, DatumType dt) : shape_(std::move(shape)), dt_(dt) {
        check(trocm_malloc(&ptr_, bytes()));
    }
    DeviceTensor(const DeviceTensor &) = delete;
    DeviceTensor &operator=(const DeviceTensor &) = delete;
    DeviceTensor(DeviceTensor &&o) noexcept { *this = std::move(o); }
    DeviceTensor &operator=(DeviceTensor &&o) noexcept {
        std::swap(ptr_, o.ptr_), std::swap(shape_, o.shape_), std::swap(dt_, o.dt_);
        return *this;
    }
    ~DeviceTensor() {
        if (ptr_) trocm_free(ptr_);
    }
    static DeviceTensor from_host(const void *host, std::vector<int64_t> shape, DatumType dt) {
        DeviceTensor t(std::move(shape), dt);
        check(trocm_h2d(t.ptr_, host, t.bytes(), nullptr));
        check(trocm_stream_sync(nullptr));
        return t;
    }
    void to_host(void *host) const {
        check(trocm_d2h(host, ptr_, bytes(), nullptr));
        check(trocm_stream_sync(nullptr));
    }
    size_t len() const {
        size_t n = 1;
        for (auto d : shape_) n *= (size_t)d;
        return n;
    }
    size_t bytes() const { return len() * size_of(dt_); }
    const std::vector<int64_t> &shape() const { return shape_; }
    DatumType datum_type() const { return dt_; }
    void *ptr() const { return ptr_; }

   private:
    void *ptr_ = nullptr;
    std::vector<int64_t> shape_;
    DatumType dt_ = DatumType::F32;
};

// Geometric-growth in-place cache along the token axis of [B, H, S, D] tensors (axis 2).
class InPlaceKvCache {
   public:
    explicit InPlaceKvCache(size_t axis, std::optional<int> storage_format = std::nullopt)
        : axis_(axis), fmt_(storage_format) {}
    InPlaceKvCache(const InPlaceKvCache &) = delete;
    InPlaceKvCache &operator=(const InPlaceKvCache &) = delete;
    InPlaceKvCache(InPlaceKvCache &&o) noexcept { *this = std::move(o); }
    InPlaceKvCache &operator=(InPlaceKvCache &&o) noexcept {
        std::swap(h_, o.h_), std::swap(axis_, o.axis_), std::swap(fmt_, o.fmt_), std::swap(shape_, o.shape_);
        std::swap(window_, o.window_);
        return *this;
    }
    // WindowKvCache::new (window_kv_cache.rs:89-93): the same object in ring-buffer mode.
    static InPlaceKvCache window(size_t axis, int64_t window, std::optional<int> storage_format = std::nullopt) {
        if (window <= 0) throw Error("window must be > 0");
        InPlaceKvCache c(axis, storage_format);
        c.window_ = window;
        return c;
    }
    int64_t cursor() const {
        if (!h_) return 0;
        int64_t w = 0, c = 0;
        check(trocm_kv_cache_window(h_, &w, &c));
        return c;
    }
    ~InPlaceKvCache() {
        if (h_) trocm_kv_cache_destroy(h_);
    }

    int64_t len() const { return get(trocm_kv_cache_len); }
    bool is_empty() const { return len() == 0; }
    int64_t capacity() const { return get(trocm_kv_cache_capacity); }
    int64_t reallocs() const { return get(trocm_kv_cache_reallocs); }

    // Append `input` along the axis, in place; O(input) amortised.
    void push(const DeviceTensor &input) {
        const auto &sh = input.shape();
        if (sh.size() != 4 || axis_ != 2) throw Error("kv-cache push: [B,H,S,D] tensors with axis 2 are supported");
        if (sh[2] == 0) return;
        if (!h_) {
            int fmt = fmt_.value_or((int)input.datum_type());
            if (window_ > 0)
                check(trocm_kv_cache_create_window(&h_, fmt, sh[0], sh[1], sh[3], window_));
            else
                check(trocm_kv_cache_create(&h_, fmt, sh[0], sh[1], sh[3]));
            shape_ = sh;
        } else if (sh[0] != shape_[0] || sh[1] != shape_[1] || sh[3] != shape_[3]) {
            throw Error("rank mismatch in kv-cache push");
        }
        int64_t strides[4] = {sh[1] * sh[2] * sh[3], sh[2] * sh[3], sh[3], 1};
        check(trocm_kv_append(h_, input.ptr(), (int)input.datum_type(), strides, sh[2], nullptr));
    }
    void truncate(int64_t len) {
        if (!h_) throw Error("Can not truncate a zero-len kv-cache value");
        check(trocm_kv_cache_truncate(h_, len));
    }
    // Dense copy of the valid [0..len] region as raw bytes (canonical block bytes when quantised).
    std::vector<uint8_t> valid_contiguous() const {
        if (!h_) throw Error("empty kv-cache");
        size_t row = 0;
        check(trocm_kv_row_bytes(h_, &row));
        size_t n = (size_t)shape_[0] * shape_[1] * (size_t)len() * row;
        void *dev = nullptr;
        check(trocm_malloc(&dev, n));
        std::vector<uint8_t> host(n);
        int rc = trocm_kv_export(h_, dev, nullptr);
        if (!rc) rc = trocm_d2h(host.data(), dev, n, nullptr);
        if (!rc) rc = trocm_stream_sync(nullptr);
        trocm_free(dev);
        check(rc);
        return host;
    }
    InPlaceKvCache clone() const {
        InPlaceKvCache c(axis_, fmt_);
        c.window_ = window_;
        if (h_) {
            check(trocm_kv_cache_clone(h_, &c.h_, nullptr));
            c.shape_ = shape_;
        }
        return c;
    }
    trocm_kv_cache *handle() const { return h_; }

   private:
    int64_t get(int (*fn)(const trocm_kv_cache *, int64_t *)) const {
        if (!h_) return 0;
        int64_t v = 0;
        check(fn(h_, &v));
        return v;
    }
    trocm_kv_cache *h_ = nullptr;
    int64_t window_ = 0;
    size_t axis_ = 2;
    std::optional<int> fmt_;
    std::vector<int64_t> shape_;
};

// Split-K scratch owned by an op state.
class Workspace {
   public:
    Workspace(int64_t batch, int64_t q_heads, int64_t q_len, int64_t head_dim) {
        check(trocm_sdpa_workspace_bytes(batch, q_heads, q_len, head_dim, &bytes_));
        check(trocm_malloc(&ptr_, bytes_));
        check(trocm_sdpa_workspace_init(ptr_, bytes_, nullptr));
    }
    Workspace(const Workspace &) = delete;
    Workspace &operator=(const Workspace &) = delete;
    ~Workspace() {
        if (ptr_) trocm_free(ptr_);
    }
    void *ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }

   private:
    void *ptr_ = nullptr;
    size_t bytes_ = 0;
};

// Scaled dot-product attention on plain device tensors.
struct Sdpa {
    std::optional<float> scale;
    bool is_causal = false;
    DeviceTensor eval(const DeviceTensor &q, const DeviceTensor &k, const DeviceTensor &v,
                      const DeviceTensor *mask = nullptr) const {
        if (is_causal && mask) throw Error("Mask cannot be provided if is_causal=true");
        const auto &qs = q.shape(), &ks = k.shape();
        if (qs.size() != 4 || ks.size() != 4 || v.shape() != ks) throw Error("Input tensors must be 4D here");
        DeviceTensor out(qs, q.datum_type());
        Workspace ws(qs[0], qs[1], qs[2], qs[3]);
        check(trocm_sdpa(q.ptr(), k.ptr(), v.ptr(), mask ? mask->ptr() : nullptr, out.ptr(), (int)q.datum_type(), qs[0],
                         qs[1], ks[1], qs[2], ks[2], qs[3], nullptr, mask ? mask->shape()[0] : 1,
                         mask ? mask->shape()[1] : 1, scale.value_or(NAN), is_causal, ws.ptr(), ws.bytes(), nullptr));
        check(trocm_stream_sync(nullptr));
        return out;
    }
};

// Fused in-place KV-cache + attention op: inputs [Q, K_new, V_new], output Q-shaped.
class InPlaceKvSdpaState {
   public:
    InPlaceKvSdpaState(size_t axis, bool causal, std::optional<float> scale, std::optional<int> fmt = std::nullopt)
        : axis_(axis), causal_(causal), scale_(scale), fmt_(fmt), k(axis, fmt), v(axis, fmt) {}

    DeviceTensor eval(const DeviceTensor &q, const DeviceTensor &k_new, const DeviceTensor &v_new) {
        k.push(k_new);
        v.push(v_new);
        const auto &qs = q.shape();
        size_t need = 0;
        check(trocm_sdpa_workspace_bytes(qs[0], qs[1], qs[2], qs[3], &need));
        if (!ws_ || ws_->bytes() < need) ws_ = std::make_unique<Workspace>(qs[0], qs[1], qs[2], qs[3]);
        DeviceTensor out(qs, q.datum_type());
        check(trocm_sdpa_cached(q.ptr(), (int)q.datum_type(), qs[1], qs[2], k.handle(), v.handle(), out.ptr(),
                                scale_.value_or(NAN), causal_, ws_->ptr(), ws_->bytes(), nullptr));
        return out;
    }
    // [K_valid, V_valid] as raw bytes; empty when nothing was pushed.
    void save_to(std::vector<std::vector<uint8_t>> &states) const {
        if (!k.is_empty()) {
            states.push_back(k.valid_contiguous());
            states.push_back(v.valid_contiguous());
        }
    }
    void load_from(const DeviceTensor &k_state, const DeviceTensor &v_state) {
        k = InPlaceKvCache(axis_, fmt_);
        v = InPlaceKvCache(axis_, fmt_);
        k.push(k_state);
        v.push(v_state);
    }
    InPlaceKvSdpaState freeze() const {
        InPlaceKvSdpaState f(axis_, causal_, scale_, fmt_);
        f.k = k.clone();
        f.v = v.clone();
        return f;
    }

   private:
    size_t axis_;
    bool causal_;
    std::optional<float> scale_;
    std::optional<int> fmt_;
    std::unique_ptr<Workspace> ws_;

   public:
    InPlaceKvCache k, v;
};

struct InPlaceKvSdpa {
    size_t axis = 2;
    bool causal = true;
    std::optional<float> scale;
    std::string name() const { return "InPlaceKvSdpa"; }
    bool is_stateless() const { return false; }
    InPlaceKvSdpaState state() const { return InPlaceKvSdpaState(axis, causal, scale); }
};

// Fused sliding-window KV-cache + attention (window_kv_cache.rs:156-239): inputs [Q, K_new, V_new].
class WindowKvSdpaState {
   public:
    WindowKvSdpaState(size_t axis, int64_t window, std::optional<float> scale, std::optional<int> fmt = std::nullopt)
        : scale_(scale), k(InPlaceKvCache::window(axis, window, fmt)), v(InPlaceKvCache::window(axis, window, fmt)) {}
    DeviceTensor eval(const DeviceTensor &q, const DeviceTensor &k_new, const DeviceTensor &v_new) {
        k.push(k_new);   // WindowKvSdpaState::eval, :224-225
        v.push(v_new);
        const auto &qs = q.shape();
        size_t need = 0;
        check(trocm_sdpa_workspace_bytes(qs[0], qs[1], qs[2], qs[3], &need));
        if (!ws_ || ws_->bytes() < need) ws_ = std::make_unique<Workspace>(qs[0], qs[1], qs[2], qs[3]);
        DeviceTensor out(qs, q.datum_type());
        // the ring buffer bounds which keys are visible: attend to all of them, no causal mask (:232-236)
        check(trocm_sdpa_cached(q.ptr(), (int)q.datum_type(), qs[1], qs[2], k.handle(), v.handle(), out.ptr(),
                                scale_.value_or(NAN), 0, ws_->ptr(), ws_->bytes(), nullptr));
        return out;
    }

   private:
    std::optional<float> scale_;
    std::unique_ptr<Workspace> ws_;

   public:
    InPlaceKvCache k, v;
};

struct WindowKvSdpa {
    size_t axis = 2;
    int64_t window = 4096;
    std::optional<float> scale;
    std::string name() const { return "WindowKvSdpa"; }
    bool is_stateless() const { return false; }
    WindowKvSdpaState state() const { return WindowKvSdpaState(axis, window, scale); }
};

// One KIVI-style quantised tensor on the device (HeadCache of every (batch, head), quant_dyn_kv_cache.rs:252-281).
class KiviCache {
   public:
    KiviCache() = default;
    KiviCache(int layout, int bits, int64_t sink_tokens, int64_t batch, int64_t heads, int64_t head_dim) {
        check(trocm_kivi_cache_create(&h_, layout, bits, sink_tokens, batch, heads, head_dim));
    }
    KiviCache(const KiviCache &) = delete;
    KiviCache &operator=(const KiviCache &) = delete;
    KiviCache(KiviCache &&o) noexcept { std::swap(h_, o.h_); }
    KiviCache &operator=(KiviCache &&o) noexcept {
        std::swap(h_, o.h_);
        return *this;
    }
    ~KiviCache() {
        if (h_) trocm_kivi_cache_destroy(h_);
    }
    bool is_some() const { return h_ != nullptr; }
    int64_t len() const {
        int64_t n = 0;
        if (h_) check(trocm_kivi_cache_len(h_, &n));
        return n;
    }
    size_t memory_bytes() const {
        size_t n = 0;
        check(trocm_kivi_cache_memory_bytes(h_, &n));
        return n;
    }
    void append(const DeviceTensor &x) {
        check(trocm_kivi_cache_append(h_, x.ptr(), (int)x.datum_type(), x.shape()[2], nullptr));
    }
    DeviceTensor dequantize(std::vector<int64_t> lead, int64_t head_dim, DatumType dt) const {
        DeviceTensor out({lead[0], lead[1], len(), head_dim}, dt);
        check(trocm_kivi_cache_dequantize(h_, out.ptr(), (int)dt, nullptr));
        return out;
    }
    KiviCache clone() const {
        KiviCache c;
        check(trocm_kivi_cache_clone(h_, &c.h_, nullptr));
        return c;
    }
    trocm_kivi_cache *handle() const { return h_; }

   private:
    trocm_kivi_cache *h_ = nullptr;
};

// quant_dyn_kv_cache.rs:334-495: the state ingests every new token and returns the whole cache, dequantised, in the
// input's datum type.  Keys (per_channel) freeze per-channel parameters per block of 32 tokens, Values quantise per
// token; the first 4 tokens stay f32.
class QuantizedDynKvCacheState {
   public:
    QuantizedDynKvCacheState(std::string name, size_t axis, uint32_t bits, bool per_channel)
        : name_(std::move(name)), axis_(axis), bits_(bits), per_channel_(per_channel) {}
    DeviceTensor eval(const DeviceTensor &input) {
        ingest(input);
        return cache_.dequantize(lead_, d_, input.datum_type());
    }
    void load_from(const DeviceTensor &init) { ingest(init); }             // :455-465
    DeviceTensor save_to() const { return cache_.dequantize(lead_, d_, DatumType::F32); }   // :467-470
    int64_t resolve_symbols() const { return cache_.len(); }              // :472-474: the past-length symbol
    QuantizedDynKvCacheState freeze() const {                            // :510-541
        QuantizedDynKvCacheState f(name_, axis_, bits_, per_channel_);
        f.lead_ = lead_, f.d_ = d_;
        if (cache_.is_some()) f.cache_ = cache_.clone();
        return f;
    }

   private:
    void ingest(const DeviceTensor &x) {                                  // :393-423
        const auto &s = x.shape();
        if (s.size() != 4) throw Error("quantized KV cache supports rank-4 [B, H, S, D] caches");
        if (axis_ != 2) throw Error("seq axis must be 2 ([B, H, S, D])");
        if (!cache_.is_some()) {
            lead_ = {s[0], s[1]}, d_ = s[3];
            cache_ = KiviCache(per_channel_ ? TROCM_KIVI_BLOCK_CHANNEL : TROCM_KIVI_PER_TOKEN, (int)bits_, 4, s[0], s[1], s[3]);
        }
        if (s[3] != d_ || s[0] != lead_[0] || s[1] != lead_[1]) throw Error("cache shape changed between steps");
        cache_.append(x);
    }
    std::string name_;
    size_t axis_;
    uint32_t bits_;
    bool per_channel_;
    std::vector<int64_t> lead_;
    int64_t d_ = 0;
    KiviCache cache_;
};

struct QuantizedDynKeyValueCache {
    std::string name;
    size_t axis = 2;
    uint32_t bits = 8;
    bool per_channel = false;
    std::string op_name() const { return "QuantizedDynKeyValueCache"; }
    bool is_stateless() const { return false; }
    QuantizedDynKvCacheState state() const {
        if (bits != 4 && bits != 8) throw Error("KV quantization bits must be 4 or 8");
        return QuantizedDynKvCacheState(name, axis, bits, per_channel);
    }
};

// kv_quant.rs:270-355: Keys in per-channel u8 with running parameters, Values in per-token u8, attention over the
// dequantised cache without a causal mask.  Inputs [Q, K_new, V_new], each [B, H, S, D].
class QuantizedKvSdpaState {
   public:
    explicit QuantizedKvSdpaState(std::optional<float> scale) : scale_(scale) {}
    DeviceTensor eval(const DeviceTensor &q, const DeviceTensor &k_new, const DeviceTensor &v_new) {
        const auto &ks = k_new.shape();
        const auto &qs = q.shape();
        if (!k.is_some()) {
            k = KiviCache(TROCM_KIVI_RUNNING_CHANNEL, 8, 0, ks[0], ks[1], ks[3]);
            v = KiviCache(TROCM_KIVI_PER_TOKEN, 8, 0, ks[0], ks[1], ks[3]);
        }
        size_t need = 0;
        check(trocm_sdpa_workspace_bytes(qs[0], qs[1], qs[2], qs[3], &need));
        if (!ws_ || ws_->bytes() < need) ws_ = std::make_unique<Workspace>(qs[0], qs[1], qs[2], qs[3]);
        DeviceTensor out(qs, q.datum_type());
        check(trocm_quantized_kv_sdpa_eval(q.ptr(), k_new.ptr(), v_new.ptr(), (int)q.datum_type(), qs[1], ks[2], k.handle(),
                                           v.handle(), out.ptr(), scale_.value_or(NAN), ws_->ptr(), ws_->bytes(), nullptr));
        return out;
    }
    QuantizedKvSdpaState freeze() const {
        QuantizedKvSdpaState f(scale_);
        if (k.is_some()) f.k = k.clone(), f.v = v.clone();
        return f;
    }

   private:
    std::optional<float> scale_;
    std::unique_ptr<Workspace> ws_;

   public:
    KiviCache k, v;
};

struct QuantizedKvSdpa {
    size_t axis = 2;
    std::optional<float> scale;
    std::string name() const { return "QuantizedKvSdpa"; }
    bool is_stateless() const { return false; }
    QuantizedKvSdpaState state() const { return QuantizedKvSdpaState(scale); }
};

// RotateHalf / ApplyRope (transformers/src/ops/apply_rope.rs:58-76, 169-176) and Cast on dense tensors;
// cos and sin share a shape that broadcasts against x (trailing-aligned).
struct RotateHalf {
    DeviceTensor eval(const DeviceTensor &x) const {
        DeviceTensor out(x.shape(), x.datum_type());
        check(trocm_rotate_half(x.ptr(), out.ptr(), (int)x.datum_type(), (int)x.shape().size(), x.shape().data(), nullptr,
                                nullptr, nullptr));
        return out;
    }
};

struct ApplyRope {
    DeviceTensor eval(const DeviceTensor &x, const DeviceTensor &cos, const DeviceTensor &sin) const {
        if (cos.shape() != sin.shape()) throw Error("cos and sin must have the same shape");
        const auto &xs = x.shape(), &cs = cos.shape();
        if (cs.size() > xs.size()) throw Error("cos/sin rank exceeds the input rank");
        std::vector<int64_t> strides(xs.size(), 0);
        int64_t acc = 1;
        for (size_t i = 0; i < xs.size(); i++) {
            size_t d = xs.size() - 1 - i;
            int64_t cd = i < cs.size() ? cs[cs.size() - 1 - i] : 1;
            if (cd != 1 && cd != xs[d]) throw Error("cos/sin shape does not broadcast against the input");
            strides[d] = (cd == 1 && xs[d] != 1) ? 0 : acc;
            acc *= cd;
        }
        DeviceTensor out(xs, x.datum_type());
        check(trocm_apply_rope(x.ptr(), cos.ptr(), sin.ptr(), out.ptr(), (int)x.datum_type(), (int)xs.size(), xs.data(),
                               nullptr, strides.data(), nullptr, nullptr));
        return out;
    }
};

struct Cast {
    DatumType to;
    DeviceTensor eval(const DeviceTensor &x) const {
        DeviceTensor out(x.shape(), to);
        check(trocm_cast(x.ptr(), (int)x.datum_type(), out.ptr(), (int)to, x.len(), nullptr));
        return out;
    }
};

// Q4_0 weights [batch, n, k] on the device and their product with a few activation rows: the
// matrix-vector arm of GgmlGemm (cuda/src/kernels/matmul/mod.rs:575-627, m <= 8).
class Q40Weights {
   public:
    // `blocks`: batch * n rows of k/32 canonical 18-byte blocks in host memory
    Q40Weights(const void *blocks, int64_t batch, int64_t n, int64_t k) : batch_(batch), n_(n), k_(k) {
        if (k % 32) throw Error("k is not a whole number of 32-element blocks");
        const size_t bytes = (size_t)batch * n * (k / 32) * 18;
        void *dev = nullptr;
        check(trocm_malloc(&dev, bytes));
        int rc = trocm_h2d(dev, blocks, bytes, nullptr);
        if (rc == 0) rc = trocm_q4_0_weights_create(&w_, dev, batch, n, k, nullptr);
        if (rc == 0) rc = trocm_stream_sync(nullptr);
        trocm_free(dev);
        check(rc);
    }
    Q40Weights(const Q40Weights &) = delete;
    Q40Weights &operator=(const Q40Weights &) = delete;
    ~Q40Weights() {
        if (w_) trocm_q4_0_weights_destroy(w_);
    }
    int64_t batch() const { return batch_; }
    int64_t n() const { return n_; }
    int64_t k() const { return k_; }
    trocm_q4_weights *handle() const { return w_; }

   private:
    trocm_q4_weights *w_ = nullptr;
    int64_t batch_, n_, k_;
};

struct GgmlGemm {
    // activations [b, m, k] (f32 or f16) x weights [b_w, n, k] -> [b, m, n]
    DeviceTensor eval(const DeviceTensor &act, const Q40Weights &w) const {
        const auto &as = act.shape();
        if (as.size() != 3 || as[2] != w.k()) throw Error("activations must be [batch, m, k]");
        DeviceTensor out({as[0], as[1], w.n()}, act.datum_type());
        check(trocm_q4_0_matvec(w.handle(), act.ptr(), (int)act.datum_type(), as[0], as[1], out.ptr(), nullptr));
        return out;
    }
};

}  // namespace trocm
