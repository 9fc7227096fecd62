// lumen.hpp -- C++17 host layer above the C ABI of liblumen_hip.so (lumen_hip.h).
//
// The reference (chen-197/Lumen) is a Rust crate; its operator API is its public
// Rust surface.  This header gives a compiled-language caller the same surface --
// the same type and function names, argument meaning and failure behaviour -- with
// every computation routed to the HIP kernels behind the C ABI.  Header-only; link
// with -llumen_hip.  Nothing here computes on the CPU.
//
//   reference (Rust)                               here (namespace lumen)
//   autograd::Tensor, no_grad, set_inference_mode  Tensor, NoGradGuard, no_grad, set_inference_mode
//   ops::matmul::matmul, Tensor + Tensor, *        ops::matmul, ops::add, ops::mul, operator+ / *
//   module::Module                                 Module
//   layers::{Linear, RMSNorm, SiLU, Embedding}     Linear, RMSNorm, SiLU, Embedding
//   layers::attention::{RotaryEmbedding,           RotaryEmbedding, KVCacheInner, KVCache,
//     KVCacheInner, KVCache, SelfAttention}          SelfAttention
//   kv_cache::LlamaKVCache                         LlamaKVCache
//   models::llama::{LlamaConfig, LlamaModel}       LlamaConfig, LlamaModel (operator by operator)
//   loader::ModelLoader::load_llama_weights        ModelLoader::load_llama_weights
//   main.rs sample_top_p + generation loop         sample_top_p, LlamaEngine::generate_turn
//   --                                             LlamaEngine: the fused model-level path
//                                                  (one HIP-graph replay per decoded token)
//
// A panic of the reference is a lumen::Error here (status() is the LUMEN_ERR_* code).
// One host thread per Context, as in the reference.
#ifndef LUMEN_HPP
#define LUMEN_HPP

#include <cstdint>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <functional>
#include <memory>
#include <numeric>
#include <optional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "lumen_hip.h"

namespace lumen {

// ----------------------------------------------------------------------------- errors
class Error : public std::runtime_error {
  public:
    Error(int status, const std::string &what) : std::runtime_error(what), status_(status) {}
    int status() const { return status_; }

  private:
    int status_;
};

inline void check(int rc) {
    if (rc != LUMEN_OK) throw Error(rc, lumen_last_error());
}

namespace detail {
[[noreturn]] __attribute__((format(printf, 2, 3))) inline void fail(int status, const char *fmt, ...) {
    char buf[256];
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    throw Error(status, buf);
}
inline size_t product(const std::vector<size_t> &s) {
    return std::accumulate(s.begin(), s.end(), (size_t)1, std::multiplies<size_t>());
}
}  // namespace detail

// ---------------------------------------------------------------------------- context
// One device, one stream (lumen_ctx).  Objects keep their context alive.
class Context {
  public:
    explicit Context(int device = 0) { check(lumen_ctx_create(device, &h_)); }
    ~Context() {
        if (h_) lumen_ctx_destroy(h_);
    }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    lumen_ctx *handle() const { return h_; }
    void synchronize() const { check(lumen_ctx_synchronize(h_)); }

    // the context used when none is given: device 0, created on first use
    static std::shared_ptr<Context> global() {
        static std::shared_ptr<Context> g = std::make_shared<Context>(0);
        return g;
    }

  private:
    lumen_ctx *h_ = nullptr;
};
using ContextPtr = std::shared_ptr<Context>;

// --------------------------------------------------------- autograd.rs:9-51 mode flags
namespace detail {
inline int &no_grad_depth() {
    thread_local int d = 0;
    return d;
}
inline bool &inference_flag() {
    thread_local bool f = false;
    return f;
}
}  // namespace detail
inline void set_inference_mode(bool on) { detail::inference_flag() = on; }          // :30
inline bool is_inference_mode() { return detail::inference_flag(); }                // :35
inline bool is_no_grad() { return detail::no_grad_depth() > 0 || is_inference_mode(); }  // :43
struct NoGradGuard {                                                                // :12-27
    NoGradGuard() { ++detail::no_grad_depth(); }
    ~NoGradGuard() { --detail::no_grad_depth(); }
    NoGradGuard(const NoGradGuard &) = delete;
    NoGradGuard &operator=(const NoGradGuard &) = delete;
};
template <class F> auto no_grad(F &&f) -> decltype(f()) {  // :48
    NoGradGuard g;
    return f();
}

// ----------------------------------------------------------------------------- Tensor
// autograd.rs:53-64: a ref-counted handle.  Here the data is an f32 array in HBM; copies
// of a Tensor and reshape() share it, like clones of the reference's Rc.  The backward
// machinery (grad, creator, backward()) is outside the inference path and absent.
class Tensor {
    struct Storage {
        ContextPtr ctx;
        void *dev = nullptr;
        size_t bytes = 0;
        Storage(ContextPtr c, size_t n) : ctx(std::move(c)), bytes(n) {
            check(lumen_malloc(ctx->handle(), n ? n : 4, &dev));
        }
        ~Storage() {
            if (dev) lumen_free(ctx->handle(), dev);
        }
        Storage(const Storage &) = delete;
        Storage &operator=(const Storage &) = delete;
    };
    struct Meta {  // shared by clones so that set_raw_data is seen through every handle
        std::shared_ptr<Storage> st;
        std::vector<size_t> shape;
    };
    std::shared_ptr<Meta> m_;

    Tensor(std::shared_ptr<Storage> st, std::vector<size_t> shape) : m_(std::make_shared<Meta>()) {
        m_->st = std::move(st);
        m_->shape = std::move(shape);
    }

  public:
    Tensor() = default;

    // Tensor::new / from_array_no_grad (:70, :161): row-major values with a shape
    static Tensor from_vec(const std::vector<float> &values, std::vector<size_t> shape, ContextPtr ctx = nullptr) {
        if (detail::product(shape) != values.size())
            detail::fail(LUMEN_ERR_SHAPE, "Tensor: %zu values for a shape of %zu elements", values.size(),
                         detail::product(shape));
        Tensor t = uninit(std::move(shape), std::move(ctx));
        if (!values.empty()) check(lumen_upload(t.ctx()->handle(), t.ptr(), values.data(), values.size() * 4));
        return t;
    }
    static Tensor zeros(std::vector<size_t> shape, ContextPtr ctx = nullptr) {
        const std::vector<float> values(detail::product(shape), 0.f);
        return from_vec(values, std::move(shape), std::move(ctx));
    }
    // device memory with no defined contents: outputs that a kernel is about to fill
    static Tensor uninit(std::vector<size_t> shape, ContextPtr ctx = nullptr) {
        if (!ctx) ctx = Context::global();
        auto st = std::make_shared<Storage>(std::move(ctx), detail::product(shape) * 4);
        return Tensor(std::move(st), std::move(shape));
    }

    bool defined() const { return (bool)m_; }
    const std::vector<size_t> &shape() const { return m_->shape; }
    size_t ndim() const { return m_->shape.size(); }
    size_t len() const { return detail::product(m_->shape); }
    const ContextPtr &ctx() const { return m_->st->ctx; }
    float *ptr() const { return (float *)m_->st->dev; }
    bool same_storage(const Tensor &o) const { return m_ && o.m_ && m_->st == o.m_->st; }

    // data() (:105): an owned host copy; waits for the stream
    std::vector<float> data() const {
        std::vector<float> out(len());
        if (!out.empty()) check(lumen_download(ctx()->handle(), out.data(), ptr(), out.size() * 4));
        return out;
    }
    std::pair<std::vector<size_t>, std::vector<float>> get_raw_data() const { return {shape(), data()}; }  // :251
    // set_raw_data (:259): replaces shape and values, visible through every clone of this handle
    void set_raw_data(std::vector<size_t> shape, const std::vector<float> &raw) {
        if (detail::product(shape) != raw.size())
            detail::fail(LUMEN_ERR_SHAPE, "set_raw_data: %zu values for a shape of %zu elements", raw.size(),
                         detail::product(shape));
        if (raw.size() * 4 > m_->st->bytes) m_->st = std::make_shared<Storage>(ctx(), raw.size() * 4);
        if (!raw.empty()) check(lumen_upload(ctx()->handle(), ptr(), raw.data(), raw.size() * 4));
        m_->shape = std::move(shape);
    }
    // fill in place from host values of the tensor's own element count (what the loader does,
    // loader.rs:44-48: the target keeps its shape)
    void assign(const float *values, size_t n) {
        if (n != len()) detail::fail(LUMEN_ERR_SHAPE, "assign: %zu values into %zu elements", n, len());
        if (n) check(lumen_upload(ctx()->handle(), ptr(), values, n * 4));
    }

    bool requires_grad() const { return false; }  // :171, inference only

    // reshape (:179, ops/shape.rs:9-49): one dimension may be -1; shares the data
    Tensor reshape(const std::vector<int> &dims) const {
        std::vector<size_t> out(dims.size());
        size_t known = 1;
        int infer = -1;
        for (size_t i = 0; i < dims.size(); ++i) {
            if (dims[i] == -1) {
                if (infer >= 0) detail::fail(LUMEN_ERR_SHAPE, "Reshape: only one dimension can be -1");
                infer = (int)i;
            } else {
                out[i] = (size_t)dims[i];
                known *= out[i];
            }
        }
        if (infer >= 0) out[infer] = known ? len() / known : 0;
        if (detail::product(out) != len())
            detail::fail(LUMEN_ERR_SHAPE, "Reshape failed: Total element count mismatch (%zu vs %zu)",
                         detail::product(out), len());
        return Tensor(m_->st, std::move(out));
    }
    // detach (:265): a new tensor with its own copy of the data
    Tensor detach() const {
        Tensor t = uninit(shape(), ctx());
        check(lumen_copy_f32(ctx()->handle(), ptr(), t.ptr(), len()));
        return t;
    }
};

// -------------------------------------------------------------------------------- ops
namespace ops {
// ops::matmul::matmul (matmul.rs:10-99): a [..., K] times b [N, K] transposed -> [..., N].
// b not 2-D or a K mismatch fails like the reference's panics (:24-38).  One row takes
// the memory-bound GEMV (:42-69), more rows the MFMA GEMM (:70-92).
inline Tensor matmul(const Tensor &a, const Tensor &b) {
    if (b.ndim() != 2) detail::fail(LUMEN_ERR_SHAPE, "MatMul RHS must be 2D, got %zu-D", b.ndim());
    if (a.ndim() == 0) detail::fail(LUMEN_ERR_SHAPE, "MatMul LHS must have at least one dimension");
    const size_t k_a = a.shape().back(), n = b.shape()[0], k_w = b.shape()[1];
    const size_t m = k_a ? a.len() / k_a : 0;
    std::vector<size_t> out_shape(a.shape().begin(), a.shape().end() - 1);
    out_shape.push_back(n);
    Tensor c = Tensor::uninit(std::move(out_shape), a.ctx());
    check(lumen_matmul_f32(a.ctx()->handle(), a.ptr(), b.ptr(), c.ptr(), (int)m, (int)n, (int)k_a, (int)k_w));
    return c;
}
namespace detail_ops {
inline void same_shape(const Tensor &a, const Tensor &b, const char *what) {
    if (a.shape() != b.shape())
        detail::fail(LUMEN_ERR_SHAPE, "%s: operand shapes differ (broadcasting is outside the inference path)", what);
}
}  // namespace detail_ops
inline Tensor add(const Tensor &a, const Tensor &b) {  // arithmetic.rs:48-51
    detail_ops::same_shape(a, b, "add");
    Tensor o = Tensor::uninit(a.shape(), a.ctx());
    check(lumen_add_f32(a.ctx()->handle(), a.ptr(), b.ptr(), o.ptr(), a.len()));
    return o;
}
inline Tensor mul(const Tensor &a, const Tensor &b) {  // arithmetic.rs:105-108
    detail_ops::same_shape(a, b, "mul");
    Tensor o = Tensor::uninit(a.shape(), a.ctx());
    check(lumen_mul_f32(a.ctx()->handle(), a.ptr(), b.ptr(), o.ptr(), a.len()));
    return o;
}
inline Tensor reshape(const Tensor &t, const std::vector<int> &dims) { return t.reshape(dims); }  // shape.rs:9
}  // namespace ops
inline Tensor operator+(const Tensor &a, const Tensor &b) { return ops::add(a, b); }
inline Tensor operator*(const Tensor &a, const Tensor &b) { return ops::mul(a, b); }

// ----------------------------------------------------------------------------- Module
struct Module {  // module.rs:12-24 (save / load of bincode checkpoints are outside the path)
    virtual ~Module() = default;
    virtual Tensor forward(Tensor input) const = 0;
    virtual std::vector<Tensor> parameters() const { return {}; }
    virtual void train_mode() { set_inference_mode(false); }
    virtual void eval_mode() { set_inference_mode(true); }
};

// linear.rs:7-50.  weight [out_features, in_features]; the inference path uses the no-bias form.
// The reference draws Kaiming-normal values at construction; here weights start at zero and
// are meant to be loaded.
class Linear : public Module {
  public:
    Tensor weight;
    static Linear new_no_bias(size_t in_features, size_t out_features, ContextPtr ctx = nullptr) {  // :25
        Linear l;
        l.weight = Tensor::zeros({out_features, in_features}, std::move(ctx));
        return l;
    }
    explicit Linear(Tensor w) : weight(std::move(w)) {}
    Tensor forward(Tensor input) const override { return ops::matmul(input, weight); }  // :33-41
    std::vector<Tensor> parameters() const override { return {weight}; }

  private:
    Linear() = default;
};

// rms_norm.rs:8-62: out = (x / sqrt(mean(x^2) + eps)) * weight over the last dimension
class RMSNorm : public Module {
  public:
    Tensor weight;
    float eps;
    RMSNorm(size_t dim, float eps_, ContextPtr ctx = nullptr)  // :14, gains start at one
        : weight(Tensor::from_vec(std::vector<float>(dim, 1.f), {dim}, std::move(ctx))), eps(eps_) {}
    Tensor forward(Tensor x) const override {
        const size_t dim = x.ndim() ? x.shape().back() : 0;
        if (dim == 0 || dim != weight.len())
            detail::fail(LUMEN_ERR_SHAPE, "RMSNorm: last dim %zu vs weight %zu", dim, weight.len());
        Tensor o = Tensor::uninit(x.shape(), x.ctx());
        check(lumen_rmsnorm_f32(x.ctx()->handle(), x.ptr(), weight.ptr(), o.ptr(), (int)(x.len() / dim), (int)dim, eps));
        return o;
    }
    std::vector<Tensor> parameters() const override { return {weight}; }
};

struct SiLU : Module {  // activation.rs:131-146
    Tensor forward(Tensor x) const override {
        Tensor o = Tensor::uninit(x.shape(), x.ctx());
        check(lumen_silu_f32(x.ctx()->handle(), x.ptr(), o.ptr(), x.len()));
        return o;
    }
};

// embedding.rs:9-57: weight [vocab, dim]; indices are f32 values (main.rs:143-152); an index
// at or beyond vocab fails (:55).  Output shape = indices shape + [dim].
class Embedding {
  public:
    Tensor weight;
    size_t vocab_size, embed_dim;
    Embedding(size_t vocab, size_t dim, ContextPtr ctx = nullptr)
        : weight(Tensor::zeros({vocab, dim}, std::move(ctx))), vocab_size(vocab), embed_dim(dim) {}
    Tensor forward(const Tensor &indices) const {
        const std::vector<float> ids = indices.data();
        std::vector<size_t> shape = indices.shape();
        shape.push_back(embed_dim);
        Tensor o = Tensor::uninit(std::move(shape), weight.ctx());
        check(lumen_embedding_f32(weight.ctx()->handle(), weight.ptr(), ids.data(), (int)ids.size(), (int)vocab_size,
                                  (int)embed_dim, o.ptr()));
        return o;
    }
    std::vector<Tensor> parameters() const { return {weight}; }
};

// ------------------------------------------------------------------------------- RoPE
// encoding.rs:6-231, half-split rotation with tables [max_seq, dim]
class RotaryEmbedding {
  public:
    size_t dim, max_seq_len;
    float theta;
    RotaryEmbedding(size_t dim_, size_t max_seq, float theta_, ContextPtr ctx = nullptr)  // :17
        : dim(dim_), max_seq_len(max_seq), theta(theta_), ctx_(ctx ? std::move(ctx) : Context::global()) {
        lumen_rope *h = nullptr;
        check(lumen_rope_create(ctx_->handle(), (int)dim, (int)max_seq, theta, &h));
        h_ = std::shared_ptr<lumen_rope>(h, [c = ctx_](lumen_rope *p) { lumen_rope_destroy(p); });
    }
    lumen_rope *handle() const { return h_.get(); }
    // forward (:56-123): x [B, H, S, D] rotated at positions offset .. offset + S - 1
    Tensor forward(const Tensor &x, size_t offset) const {
        if (x.ndim() != 4) detail::fail(LUMEN_ERR_SHAPE, "RoPE input must be [B, H, S, D], got %zu-D", x.ndim());
        const auto &s = x.shape();
        Tensor o = Tensor::uninit(s, x.ctx());
        check(lumen_rope_forward_f32(h_.get(), x.ptr(), o.ptr(), (int)s[0], (int)s[1], (int)s[2], (int)s[3], (int)offset));
        return o;
    }
    // rope_1token_copy (:173-204) on device vectors of length dim
    void rope_1token_copy(const Tensor &src, Tensor &dst, size_t pos) const {
        if (src.len() != dst.len()) detail::fail(LUMEN_ERR_SHAPE, "rope_1token_copy: src %zu vs dst %zu", src.len(), dst.len());
        check(lumen_rope_1token_copy_f32(h_.get(), src.ptr(), dst.ptr(), (int)src.len(), (int)pos));
    }
    // the same on host slices, as the reference's signature has it
    void rope_1token_copy(const std::vector<float> &src, std::vector<float> &dst, size_t pos) const {
        Tensor s = Tensor::from_vec(src, {src.size()}, ctx_), d = Tensor::uninit({src.size()}, ctx_);
        rope_1token_copy(s, d, pos);
        dst = d.data();
    }
    // cos_sin_row_vec (:208-229)
    std::pair<std::vector<float>, std::vector<float>> cos_sin_row_vec(size_t pos) const {
        if (pos >= max_seq_len)
            detail::fail(LUMEN_ERR_ROPE_RANGE, "RoPE index out of range: pos %zu >= max %zu", pos, max_seq_len);
        std::vector<float> c(max_seq_len * dim), s(max_seq_len * dim);
        check(lumen_rope_tables_download(h_.get(), c.data(), s.data()));
        return {std::vector<float>(c.begin() + pos * dim, c.begin() + (pos + 1) * dim),
                std::vector<float>(s.begin() + pos * dim, s.begin() + (pos + 1) * dim)};
    }

  private:
    ContextPtr ctx_;
    std::shared_ptr<lumen_rope> h_;
};

// --------------------------------------------------------------------------- KV cache
// self_attention.rs:24-44: k, v [B, H_kv, max_seq, D] zero-initialised in HBM, plus len
class KVCacheInner {
  public:
    KVCacheInner(size_t b, size_t h_kv, size_t max_seq, size_t d, ContextPtr ctx = nullptr)  // :33
        : shape_{b, h_kv, max_seq, d}, ctx_(ctx ? std::move(ctx) : Context::global()) {
        check(lumen_kv_cache_create(ctx_->handle(), (int)b, (int)h_kv, (int)max_seq, (int)d, &h_));
    }
    ~KVCacheInner() {
        if (h_) lumen_kv_cache_destroy(h_);
    }
    KVCacheInner(const KVCacheInner &) = delete;
    KVCacheInner &operator=(const KVCacheInner &) = delete;
    void reset() { check(lumen_kv_cache_reset(h_)); }  // :41-43: len = 0, data kept
    size_t len() const {
        int n = 0;
        check(lumen_kv_cache_len(h_, &n));
        return (size_t)n;
    }
    void set_len(size_t n) { check(lumen_kv_cache_set_len(h_, (int)n)); }  // a public field in the reference (:28)
    const std::vector<size_t> &shape() const { return shape_; }
    std::vector<float> k() const { return download(true); }
    std::vector<float> v() const { return download(false); }
    lumen_kv_cache *handle() const { return h_; }
    const ContextPtr &ctx() const { return ctx_; }

  private:
    std::vector<float> download(bool want_k) const {
        float *kp = nullptr, *vp = nullptr;
        check(lumen_kv_cache_ptrs(h_, &kp, &vp));
        std::vector<float> out(detail::product(shape_));
        check(lumen_download(ctx_->handle(), out.data(), want_k ? kp : vp, out.size() * 4));
        return out;
    }
    std::vector<size_t> shape_;
    ContextPtr ctx_;
    lumen_kv_cache *h_ = nullptr;
};
using KVCache = std::shared_ptr<KVCacheInner>;  // :30, Rc<RefCell<KVCacheInner>>

// kv_cache.rs:5-60, the older cache type: explicit start position, copied-out views
class LlamaKVCache {
  public:
    size_t max_seq_len, head_num, dim;
    LlamaKVCache(size_t max_seq, size_t kv_heads, size_t head_dim, ContextPtr ctx = nullptr)
        : max_seq_len(max_seq), head_num(kv_heads), dim(head_dim), inner_(1, kv_heads, max_seq, head_dim, std::move(ctx)) {}
    void update(const Tensor &k, const Tensor &v, size_t start_pos) {  // :31-49, k / v [1, H_kv, S, D]
        if (k.ndim() != 4 || k.shape() != v.shape()) detail::fail(LUMEN_ERR_SHAPE, "LlamaKVCache::update: k, v must be [1, H_kv, S, D]");
        check(lumen_kv_cache_update(inner_.handle(), k.ptr(), v.ptr(), (int)k.shape()[2], (int)start_pos));
    }
    std::pair<Tensor, Tensor> get_view(size_t current_len) const {  // :51-59
        Tensor k = Tensor::uninit({1, head_num, current_len, dim}, inner_.ctx());
        Tensor v = Tensor::uninit({1, head_num, current_len, dim}, inner_.ctx());
        check(lumen_kv_cache_get_view(inner_.handle(), (int)current_len, k.ptr(), v.ptr()));
        return {k, v};
    }

  private:
    KVCacheInner inner_;
};

// ---------------------------------------------------------------------- SelfAttention
// self_attention.rs:46-470, the two inference paths: decode (S == 1, :125-306) and
// prefill (S > 1, :308-427).  The training path (:429-469) is outside this build.
class SelfAttention : public Module {
  public:
    Linear w_q, w_k, w_v, w_o;
    RotaryEmbedding rope;
    size_t n_head, n_kv_head, head_dim, max_seq;
    float scale;
    bool causal;

    SelfAttention(size_t embed_dim, size_t n_head_, size_t n_kv_head_, size_t max_seq_len, float rope_theta,
                  bool causal_, ContextPtr ctx = nullptr)  // :61-94
        : SelfAttention(checked_dims(embed_dim, n_head_, n_kv_head_), embed_dim, n_head_, n_kv_head_, max_seq_len,
                        rope_theta, causal_, ctx ? std::move(ctx) : Context::global()) {}

    // x [B, S, E]; returns (out [B, S, E], the cache that now holds S more positions)
    std::pair<Tensor, std::optional<KVCache>> forward(Tensor x, std::optional<KVCache> cache) const {  // :96
        if (x.ndim() != 3) detail::fail(LUMEN_ERR_SHAPE, "SelfAttention input must be [B, S, E], got %zu-D", x.ndim());
        if (!is_no_grad())
            detail::fail(LUMEN_ERR_UNSUPPORTED, "SelfAttention: the training path is outside this build; "
                                                "enter no_grad or set_inference_mode(true)");
        const size_t b = x.shape()[0], s = x.shape()[1];
        Tensor q = w_q.forward(x), k = w_k.forward(x), v = w_v.forward(x);  // :106-108
        KVCache c = cache ? *cache : std::make_shared<KVCacheInner>(b, n_kv_head, max_seq, head_dim, x.ctx());  // :119-122
        Tensor att = Tensor::uninit({b, s, n_head, head_dim}, x.ctx());
        if (s == 1)
            check(lumen_attn_decode_f32(c->handle(), rope.handle(), q.ptr(), k.ptr(), v.ptr(), att.ptr(), (int)n_head,
                                        scale, causal));
        else
            check(lumen_attn_prefill_f32(c->handle(), rope.handle(), q.ptr(), k.ptr(), v.ptr(), att.ptr(), (int)s,
                                         (int)n_head, scale, causal));
        Tensor out = w_o.forward(att.reshape({(int)b, (int)s, (int)(n_head * head_dim)}));  // :300-303, :421-424
        return {out, c};
    }
    Tensor forward(Tensor x) const override { return forward(std::move(x), std::nullopt).first; }
    std::vector<Tensor> parameters() const override { return {w_q.weight, w_k.weight, w_v.weight, w_o.weight}; }

  private:
    static size_t checked_dims(size_t embed_dim, size_t n_head, size_t n_kv_head) {
        if (n_head == 0 || embed_dim % n_head) detail::fail(LUMEN_ERR_SHAPE, "Embed dim must be divisible by n_head");  // :69-73
        if (n_kv_head == 0 || n_head % n_kv_head) detail::fail(LUMEN_ERR_SHAPE, "n_head must be divisible by n_kv_head");
        return embed_dim / n_head;
    }
    SelfAttention(size_t d, size_t e, size_t h, size_t hkv, size_t max_seq_len, float theta, bool causal_, ContextPtr ctx)
        : w_q(Linear::new_no_bias(e, e, ctx)), w_k(Linear::new_no_bias(e, hkv * d, ctx)),
          w_v(Linear::new_no_bias(e, hkv * d, ctx)), w_o(Linear::new_no_bias(e, e, ctx)),
          rope(d, max_seq_len, theta, ctx), n_head(h), n_kv_head(hkv), head_dim(d), max_seq(max_seq_len),
          scale(1.0f / std::sqrt((float)d)), causal(causal_) {}  // :89
};

// ------------------------------------------------------------------------------ Llama
struct LlamaConfig {  // llama.rs:11-37 (defaults: TinyLlama-1.1B)
    size_t vocab_size = 32000, hidden_size = 2048, intermediate_size = 5632, num_hidden_layers = 22;
    size_t num_attention_heads = 32, num_key_value_heads = 4;
    float rms_norm_eps = 1e-5f;
    size_t max_seq_len = 2048;
    float rope_theta = 10000.0f;
};

class LlamaMLP : public Module {  // llama.rs:40-66: down(silu(gate(x)) * up(x)), five operator calls
  public:
    Linear gate_proj, up_proj, down_proj;
    SiLU act;
    LlamaMLP(const LlamaConfig &c, const ContextPtr &ctx)
        : gate_proj(Linear::new_no_bias(c.hidden_size, c.intermediate_size, ctx)),
          up_proj(Linear::new_no_bias(c.hidden_size, c.intermediate_size, ctx)),
          down_proj(Linear::new_no_bias(c.intermediate_size, c.hidden_size, ctx)) {}
    Tensor forward(Tensor x) const override {
        Tensor gate_act = act.forward(gate_proj.forward(x));
        Tensor fused = gate_act * up_proj.forward(x);
        return down_proj.forward(fused);
    }
    std::vector<Tensor> parameters() const override { return {gate_proj.weight, up_proj.weight, down_proj.weight}; }
};

class LlamaDecoderLayer {  // llama.rs:79-116
  public:
    SelfAttention self_attn;
    LlamaMLP mlp;
    RMSNorm input_layernorm, post_attention_layernorm;
    LlamaDecoderLayer(const LlamaConfig &c, const ContextPtr &ctx)
        : self_attn(c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.max_seq_len, c.rope_theta, true, ctx),
          mlp(c, ctx), input_layernorm(c.hidden_size, c.rms_norm_eps, ctx),
          post_attention_layernorm(c.hidden_size, c.rms_norm_eps, ctx) {}
    std::pair<Tensor, KVCache> forward_infer(const Tensor &x, KVCache cache) const {  // :104-116, pre-norm
        auto [attn_out, cache_out] = self_attn.forward(input_layernorm.forward(x), std::move(cache));
        Tensor h = x + attn_out;
        Tensor mlp_out = mlp.forward(post_attention_layernorm.forward(h));
        return {h + mlp_out, *cache_out};
    }
};

// llama.rs:129-280: the network composed operator by operator, one C-ABI call per reference
// operator.  For generation speed hand it to LlamaEngine below.
class LlamaModel {
  public:
    LlamaConfig config;
    Embedding embed_tokens;
    std::vector<LlamaDecoderLayer> layers;
    RMSNorm norm;
    Linear lm_head;

    explicit LlamaModel(const LlamaConfig &c, ContextPtr ctx = nullptr)  // :138-159
        : LlamaModel(c, ctx ? std::move(ctx) : Context::global(), 0) {}

    std::vector<KVCache> init_kv_caches(size_t batch_size) const {  // :161-169
        std::vector<KVCache> out;
        const size_t d = config.hidden_size / config.num_attention_heads;
        for (size_t i = 0; i < config.num_hidden_layers; ++i)
            out.push_back(std::make_shared<KVCacheInner>(batch_size, config.num_key_value_heads, config.max_seq_len, d, ctx_));
        return out;
    }
    void reset_kv_caches(std::vector<KVCache> &caches) const {  // :172-176
        for (auto &c : caches) c->reset();
    }
    // forward (:181-206): ids [B, S] as f32 -> logits [B, S, V]; the position comes from the caches
    Tensor forward(const Tensor &input_ids, std::vector<KVCache> &caches, size_t /*pos*/ = 0) const {
        if (caches.size() != layers.size())
            detail::fail(LUMEN_ERR_CACHE_COUNT, "KV cache count mismatch: got %zu, expected %zu", caches.size(), layers.size());
        Tensor x = embed_tokens.forward(input_ids);
        for (size_t i = 0; i < layers.size(); ++i) {
            auto [y, cache_out] = layers[i].forward_infer(x, caches[i]);
            caches[i] = cache_out;
            x = y;
        }
        return lm_head.forward(norm.forward(x));
    }
    // named_parameters (:218-279): HF tensor names -> handles sharing the model's data
    std::unordered_map<std::string, Tensor> named_parameters() const {
        std::unordered_map<std::string, Tensor> p;
        p["model.embed_tokens.weight"] = embed_tokens.weight;
        for (size_t i = 0; i < layers.size(); ++i) {
            const std::string pre = "model.layers." + std::to_string(i);
            const LlamaDecoderLayer &l = layers[i];
            p[pre + ".self_attn.q_proj.weight"] = l.self_attn.w_q.weight;
            p[pre + ".self_attn.k_proj.weight"] = l.self_attn.w_k.weight;
            p[pre + ".self_attn.v_proj.weight"] = l.self_attn.w_v.weight;
            p[pre + ".self_attn.o_proj.weight"] = l.self_attn.w_o.weight;
            p[pre + ".mlp.gate_proj.weight"] = l.mlp.gate_proj.weight;
            p[pre + ".mlp.up_proj.weight"] = l.mlp.up_proj.weight;
            p[pre + ".mlp.down_proj.weight"] = l.mlp.down_proj.weight;
            p[pre + ".input_layernorm.weight"] = l.input_layernorm.weight;
            p[pre + ".post_attention_layernorm.weight"] = l.post_attention_layernorm.weight;
        }
        p["model.norm.weight"] = norm.weight;
        p["lm_head.weight"] = lm_head.weight;
        return p;
    }
    std::vector<Tensor> parameters() const {  // :289-309, the order of the reference's list
        std::vector<Tensor> p{embed_tokens.weight};
        for (const auto &l : layers) {
            for (const Tensor &t : l.self_attn.parameters()) p.push_back(t);
            for (const Tensor &t : l.mlp.parameters()) p.push_back(t);
            p.push_back(l.input_layernorm.weight);
            p.push_back(l.post_attention_layernorm.weight);
        }
        p.push_back(norm.weight);
        p.push_back(lm_head.weight);
        return p;
    }
    const ContextPtr &ctx() const { return ctx_; }

  private:
    LlamaModel(const LlamaConfig &c, ContextPtr ctx, int)
        : config(c), embed_tokens(c.vocab_size, c.hidden_size, ctx), norm(c.hidden_size, c.rms_norm_eps, ctx),
          lm_head(Linear::new_no_bias(c.hidden_size, c.vocab_size, ctx)), ctx_(std::move(ctx)) {
        layers.reserve(c.num_hidden_layers);
        for (size_t i = 0; i < c.num_hidden_layers; ++i) layers.emplace_back(c, ctx_);
    }
    ContextPtr ctx_;
};

// ----------------------------------------------------------------------------- loader
struct ModelLoader {
    // load_llama_weights (loader.rs:10-80): fills every tensor of model_params that the
    // .safetensors file holds (F32, or BF16 widened to f32), keeping the target's shape; an
    // element count that differs fails ("Shape mismatch for ..."), another dtype fails
    // ("Unsupported dtype"), a name the file lacks is skipped and counted (the reference warns).
    // Returns {tensors loaded, names missing}.
    static std::pair<int, int> load_llama_weights(const std::string &path,
                                                  const std::unordered_map<std::string, Tensor> &model_params) {
        std::FILE *f = std::fopen(path.c_str(), "rb");
        if (!f) detail::fail(LUMEN_ERR_INVALID, "cannot open %s", path.c_str());
        struct Closer {
            std::FILE *f;
            ~Closer() { std::fclose(f); }
        } closer{f};
        unsigned char len8[8];
        if (std::fread(len8, 1, 8, f) != 8) detail::fail(LUMEN_ERR_INVALID, "%s: no safetensors header", path.c_str());
        uint64_t header_len = 0;
        for (int i = 7; i >= 0; --i) header_len = (header_len << 8) | len8[i];
        int loaded = 0, missing = 0;
        std::vector<unsigned char> raw;
        std::vector<float> vals;
        for (const auto &[name, target] : model_params) {
            int dtype = -1, ndim = 8;
            int64_t shape[8];
            uint64_t begin = 0, end = 0;
            if (lumen_safetensors_find(path.c_str(), name.c_str(), &dtype, shape, &ndim, &begin, &end) != LUMEN_OK) {
                ++missing;
                continue;
            }
            if (dtype != LUMEN_DTYPE_F32 && dtype != LUMEN_DTYPE_BF16)
                detail::fail(LUMEN_ERR_INVALID, "Unsupported dtype for %s", name.c_str());
            const size_t esz = dtype == LUMEN_DTYPE_F32 ? 4 : 2, n = (size_t)(end - begin) / esz;
            if (n != target.len())
                detail::fail(LUMEN_ERR_SHAPE, "Shape mismatch for %s: %zu elements in the file, %zu in the model",
                             name.c_str(), n, target.len());
            raw.resize(n * esz);
            if (std::fseek(f, (long)(8 + header_len + begin), SEEK_SET) != 0 || std::fread(raw.data(), 1, raw.size(), f) != raw.size())
                detail::fail(LUMEN_ERR_INVALID, "%s: short read of %s", path.c_str(), name.c_str());
            if (dtype == LUMEN_DTYPE_F32) {
                Tensor(target).assign((const float *)raw.data(), n);
            } else {  // loader.rs:50-64: bf16 -> f32 is the bit pattern shifted up 16
                vals.resize(n);
                for (size_t i = 0; i < n; ++i) {
                    const uint32_t bits = (uint32_t)(raw[2 * i] | (raw[2 * i + 1] << 8)) << 16;
                    std::memcpy(&vals[i], &bits, 4);
                }
                Tensor(target).assign(vals.data(), n);
            }
            ++loaded;
        }
        return {loaded, missing};
    }
};

// ---------------------------------------------------------------------------- sampler
// sample_top_p (main.rs:74-137) with the uniform draw r given by the caller
inline int32_t sample_top_p(const std::vector<float> &logits, float temperature, float top_p, float repetition_penalty,
                            const std::vector<int32_t> &recent_tokens, float r) {
    int32_t pick = 0;
    check(lumen_sample_top_p_f32(logits.data(), (int)logits.size(), temperature, top_p, repetition_penalty,
                                 recent_tokens.data(), (int)recent_tokens.size(), r, &pick));
    return pick;
}

// LlamaDecoderLayer::forward_infer for ONE token as one operator call (llama.rs:104-116 behind
// lumen_decoder_layer_decode_f32): the launches of the model-level decode step -- three per layer where the chained
// launch covers the shape -- for an integration that replaces the reference layer by layer.  One object serves every
// layer of a stack; weights in the fused layouts (q|k|v rows one after the other, gate / up rows interleaved:
// lumen_interleave_rows).  No counterpart in the reference.
class DecoderLayerStep {
  public:
    DecoderLayerStep(const lumen_llama_config &cfg, ContextPtr ctx = nullptr) : ctx_(ctx ? std::move(ctx) : Context::global()) {
        check(lumen_decoder_layer_create(ctx_->handle(), &cfg, &h_));
    }
    ~DecoderLayerStep() {
        if (h_) lumen_decoder_layer_destroy(h_);
    }
    DecoderLayerStep(const DecoderLayerStep &) = delete;
    DecoderLayerStep &operator=(const DecoderLayerStep &) = delete;
    // y = layer(x) for the token at position cache.len; the cache length advances by one
    void decode(KVCacheInner &cache, const Tensor &wqkv, const Tensor &wo, const Tensor &wgu, const Tensor &wdown,
                const Tensor &input_norm, const Tensor &post_norm, const Tensor &x, Tensor &y) {
        check(lumen_decoder_layer_decode_f32(h_, cache.handle(), wqkv.ptr(), wo.ptr(), wgu.ptr(), wdown.ptr(), input_norm.ptr(),
                                             post_norm.ptr(), nullptr, nullptr, x.ptr(), y.ptr()));
    }

  private:
    ContextPtr ctx_;
    lumen_decoder_layer *h_ = nullptr;
};

// ----------------------------------------------------------------------------- engine
// No counterpart in the reference: the same network as LlamaModel with its weights in fused
// layouts (q|k|v rows concatenated, gate/up rows interleaved), five kernels per layer and one
// HIP-graph replay per decoded token.  Built from a LlamaModel's current parameter values (a
// copy: later changes to the model's tensors are not seen) or filled by name / from a file.
class LlamaEngine {
  public:
    explicit LlamaEngine(const lumen_llama_config &cfg, ContextPtr ctx = nullptr)
        : ctx_(ctx ? std::move(ctx) : Context::global()), cfg_(cfg) {
        check(lumen_llama_create(ctx_->handle(), &cfg_, &h_));
    }
    explicit LlamaEngine(const LlamaModel &m) : LlamaEngine(to_c_config(m.config), m.ctx()) {
        for (const auto &[name, t] : m.named_parameters()) set_param(name, t.data(), t.shape());
    }
    ~LlamaEngine() {
        if (h_) lumen_llama_destroy(h_);
    }
    LlamaEngine(const LlamaEngine &) = delete;
    LlamaEngine &operator=(const LlamaEngine &) = delete;

    static lumen_llama_config to_c_config(const LlamaConfig &c) {
        lumen_llama_config o{};
        o.vocab_size = (int)c.vocab_size;
        o.hidden_size = (int)c.hidden_size;
        o.intermediate_size = (int)c.intermediate_size;
        o.num_hidden_layers = (int)c.num_hidden_layers;
        o.num_attention_heads = (int)c.num_attention_heads;
        o.num_key_value_heads = (int)c.num_key_value_heads;
        o.rms_norm_eps = c.rms_norm_eps;
        o.max_seq_len = (int)c.max_seq_len;
        o.rope_theta = c.rope_theta;
        o.weight_dtype = LUMEN_DTYPE_F32;
        return o;
    }
    void set_param(const std::string &name, const std::vector<float> &values, const std::vector<size_t> &shape) {
        std::vector<int64_t> s(shape.begin(), shape.end());
        check(lumen_llama_set_param(h_, name.c_str(), values.data(), LUMEN_DTYPE_F32, s.data(), (int)s.size()));
    }
    std::pair<int, int> load_safetensors(const std::string &path) {  // loader.rs:10-80
        int loaded = 0, missing = 0;
        check(lumen_llama_load_safetensors(h_, path.c_str(), &loaded, &missing));
        return {loaded, missing};
    }
    // LlamaModel::forward (llama.rs:181-206) on the engine's own caches: ids as f32; returns the
    // logits of every position [S * V] (all_rows, what the reference computes) or of the last one [V]
    std::vector<float> forward(const std::vector<float> &ids, bool all_rows = false) {
        std::vector<float> logits((all_rows ? ids.size() : 1) * (size_t)cfg_.vocab_size);
        check(lumen_llama_forward(h_, ids.data(), (int)ids.size(), logits.data(), all_rows));
        return logits;
    }
    // the generation loop of main.rs:340-378 with greedy picks, without leaving the GPU
    std::vector<int32_t> decode_greedy(int32_t first_id, int n) {
        std::vector<int32_t> out((size_t)n);
        check(lumen_llama_decode_greedy(h_, first_id, n, out.data(), nullptr));
        return out;
    }
    // one chat turn (main.rs:325-378) with top-p sampling from a seeded stream
    std::vector<int32_t> generate_turn(const std::vector<int32_t> &new_tokens, const std::vector<int32_t> &history,
                                       const lumen_sampling &sampling, const std::vector<int32_t> &stop_ids) {
        std::vector<int32_t> out((size_t)(sampling.max_gen > 0 ? sampling.max_gen : 1));
        int n = 0;
        check(lumen_llama_generate_turn(h_, new_tokens.data(), (int)new_tokens.size(), history.data(), (int)history.size(),
                                        &sampling, stop_ids.data(), (int)stop_ids.size(), out.data(), (int)out.size(), &n));
        out.resize((size_t)n);
        return out;
    }
    void reset_kv_caches() { check(lumen_llama_reset(h_)); }  // llama.rs:172-176
    void set_kv_len(size_t n) { check(lumen_llama_set_kv_len(h_, (int)n)); }  // KVCacheInner.len, a public field (:28)
    size_t kv_len() const {
        int n = 0;
        check(lumen_llama_kv_len(h_, &n));
        return (size_t)n;
    }
    lumen_llama *handle() const { return h_; }
    const lumen_llama_config &config() const { return cfg_; }

  private:
    ContextPtr ctx_;
    lumen_llama_config cfg_;
    lumen_llama *h_ = nullptr;
};

}  // namespace lumen
#endif
