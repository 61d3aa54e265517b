// fusor_hip.hpp -- C++ host side above the C ABI of fusor_hip.h.
//
// Header-only mirror of the fusor types that sit on the attention path, with the reference's
// names, argument order and failure behaviour, so code written against
//     fusor::Tensor<4, D>::flash_attention(&k, &v, scale, Option<(&mask, MaskKind)>)
//                                   fusor-ml/fusor/src/composite/flash_attention.rs:52-73
//     fusor::cache::{AttentionMask, MaskCache, KvCache}
//                                   fusor-ml/fusor/src/cache/{attention_mask,mask_cache,kv_cache}.rs
// reads the same here.  Where the reference panics (assert!/panic!) these functions throw
// fusor_hip::Panic carrying the reference's message; HIP failures throw fusor_hip::GpuError (the
// reference's fusor::Error::Gpu, fusor-ml/fusor/src/lib.rs:391-403).
// Tensors are reference-counted views {buffer, offset, shape, strides} in element units
// (fusor-ml/types/src/layout.rs:88-129); layout operations never copy.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "fusor_hip.h"

namespace fusor_hip {

struct Panic : std::logic_error {
    using std::logic_error::logic_error;
};
struct GpuError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

inline void check(int status) {
    if (status == FHIP_OK) return;
    const std::string msg = fhip_last_error();
    if (status == FHIP_ERR_INVALID_ARG) throw Panic(msg);
    throw GpuError(msg);
}

enum class DType { F32 = FHIP_F32, F16 = FHIP_F16, BF16 = FHIP_BF16 };
inline size_t dtype_bytes(DType d) { return d == DType::F32 ? 4 : 2; }

/// fusor::MaskKind (flash_attention.rs:11-19)
enum class MaskKind { QKMask = FHIP_MASK_QK, BatchKeyMask = FHIP_MASK_BATCH_KEY };

/// One GPU plus one stream.  Cheap to copy (shared handle), like fusor's Device.
/// A recorded sequence of library calls (fhip_graph); launch() replays it with one submission.
class Graph {
    struct Inner {
        fhip_graph *g = nullptr;
        ~Inner() {
            if (g) fhip_graph_destroy(g);
        }
    };
    std::shared_ptr<Inner> in_;
    fhip_stream *stream_;

   public:
    Graph(fhip_graph *g, fhip_stream *s) : in_(std::make_shared<Inner>()), stream_(s) { in_->g = g; }
    void launch() const { check(fhip_graph_launch(in_->g, stream_)); }
};

class Device {
    struct Inner {
        fhip_device *dev = nullptr;
        fhip_stream *stream = nullptr;
        fhip_device_info info{};
        void *workspace = nullptr;
        size_t workspace_bytes = 0;
        ~Inner() {
            if (workspace) fhip_free(dev, workspace);
            if (stream) fhip_stream_destroy(stream);
            if (dev) fhip_device_destroy(dev);
        }
    };
    std::shared_ptr<Inner> in_;

   public:
    explicit Device(int ordinal = 0) : in_(std::make_shared<Inner>()) {
        check(fhip_device_create(ordinal, &in_->dev));
        check(fhip_stream_create(in_->dev, &in_->stream));
        check(fhip_device_get_info(in_->dev, &in_->info));
    }
    fhip_device *handle() const { return in_->dev; }
    fhip_stream *stream() const { return in_->stream; }
    const fhip_device_info &info() const { return in_->info; }
    void synchronize() const { check(fhip_stream_synchronize(in_->stream)); }
    bool same(const Device &o) const { return in_ == o.in_; }
    /// grow-only scratch for the split-KV decode (the caller of the C ABI owns the workspace)
    void *workspace(size_t bytes) const {
        if (bytes > in_->workspace_bytes) {
            if (in_->workspace) {
                synchronize();
                check(fhip_free(in_->dev, in_->workspace));
                in_->workspace = nullptr;
            }
            check(fhip_malloc(in_->dev, bytes, &in_->workspace));
            in_->workspace_bytes = bytes;
        }
        return in_->workspace;
    }
    size_t workspace_bytes() const { return in_->workspace_bytes; }
    /// Records the library calls `body` makes on this device's stream instead of running them.  The body must not
    /// allocate or read back (pre-allocate outputs and workspace; no as_slice / to_host inside).
    template <typename F>
    Graph capture(F &&body) const {
        check(fhip_stream_begin_capture(in_->stream));
        try {
            body();
        } catch (...) {
            fhip_graph *dropped = nullptr;
            (void)fhip_stream_end_capture(in_->stream, &dropped);
            if (dropped) fhip_graph_destroy(dropped);
            throw;
        }
        fhip_graph *g = nullptr;
        check(fhip_stream_end_capture(in_->stream, &g));
        return Graph(g, in_->stream);
    }
};

/// Owning device allocation, freed with the last tensor that views it.
class Buffer {
    Device dev_;
    void *ptr_ = nullptr;
    bool owned_ = true;

   public:
    Buffer(const Device &dev, size_t bytes) : dev_(dev) { check(fhip_malloc(dev.handle(), bytes, &ptr_)); }
    Buffer(const Device &dev, void *borrowed) : dev_(dev), ptr_(borrowed), owned_(false) {}
    Buffer(const Buffer &) = delete;
    Buffer &operator=(const Buffer &) = delete;
    ~Buffer() {
        if (owned_ && ptr_) fhip_free(dev_.handle(), ptr_);
    }
    void *ptr() const { return ptr_; }
    const Device &device() const { return dev_; }
};

/// Rank-R strided view of device memory.
template <int R>
class Tensor {
    std::shared_ptr<Buffer> buf_;
    std::shared_ptr<void> keepalive_;  // e.g. the KV cache that owns a borrowed buffer
    DType dtype_ = DType::F32;
    uint64_t offset_ = 0;
    uint32_t shape_[R]{};
    int64_t stride_[R]{};

   public:
    Tensor() = default;
    Tensor(std::shared_ptr<Buffer> buf, DType dt, const uint32_t (&shape)[R], const int64_t *strides = nullptr,
           uint64_t offset = 0, std::shared_ptr<void> keepalive = nullptr)
        : buf_(std::move(buf)), keepalive_(std::move(keepalive)), dtype_(dt), offset_(offset) {
        int64_t acc = 1;
        for (int i = R - 1; i >= 0; i--) {
            shape_[i] = shape[i];
            stride_[i] = strides ? strides[i] : acc;
            acc *= shape[i];
        }
    }
    /// Tensor::zeros-like allocation without initialisation (the kernels overwrite it)
    static Tensor empty(const Device &dev, DType dt, const uint32_t (&shape)[R]) {
        size_t n = 1;
        for (int i = 0; i < R; i++) n *= shape[i];
        return Tensor(std::make_shared<Buffer>(dev, n * dtype_bytes(dt)), dt, shape);
    }
    /// Tensor::from_slice: uploads contiguous host elements of the tensor's dtype
    static Tensor from_slice(const Device &dev, DType dt, const uint32_t (&shape)[R], const void *host) {
        Tensor t = empty(dev, dt, shape);
        check(fhip_memcpy_h2d(dev.stream(), t.buf_->ptr(), host, t.numel() * dtype_bytes(dt)));
        return t;
    }
    size_t numel() const {
        size_t n = 1;
        for (int i = 0; i < R; i++) n *= shape_[i];
        return n;
    }
    const uint32_t *shape() const { return shape_; }
    const int64_t *strides() const { return stride_; }
    uint64_t offset() const { return offset_; }
    DType dtype() const { return dtype_; }
    const Device &device() const { return buf_->device(); }
    void *data() const { return buf_->ptr(); }
    bool is_contiguous() const {
        int64_t acc = 1;
        for (int i = R - 1; i >= 0; i--) {
            if (shape_[i] != 1 && stride_[i] != acc) return false;
            acc *= shape_[i];
        }
        return true;
    }
    /// Layout::transpose (types/src/layout.rs): swaps two dimensions, no copy
    Tensor transpose(int a, int b) const {
        Tensor t = *this;
        std::swap(t.shape_[a], t.shape_[b]);
        std::swap(t.stride_[a], t.stride_[b]);
        return t;
    }
    /// Layout::narrow: a window along one dimension, no copy
    Tensor narrow(int dim, uint32_t start, uint32_t len) const {
        if (start + (uint64_t)len > shape_[dim]) throw Panic("narrow out of range");
        Tensor t = *this;
        t.shape_[dim] = len;
        t.offset_ += (uint64_t)start * (uint64_t)stride_[dim];
        return t;
    }
    /// Layout::broadcast_to: dimensions of size 1 repeat with stride 0, no copy
    Tensor broadcast_to(const uint32_t (&shape)[R]) const {
        Tensor t = *this;
        for (int i = 0; i < R; i++) {
            if (shape_[i] == shape[i]) continue;
            if (shape_[i] != 1) throw Panic("broadcast_to: only dimensions of size 1 repeat");
            t.shape_[i] = shape[i];
            t.stride_[i] = 0;
        }
        return t;
    }
    /// as_slice().await: contiguous readback of this view (synchronises the stream)
    void to_host(void *host) const {
        if (!is_contiguous()) throw Panic("to_host needs a contiguous view");
        const size_t eb = dtype_bytes(dtype_);
        check(fhip_memcpy_d2h(device().stream(), host, (const char *)buf_->ptr() + offset_ * eb, numel() * eb));
    }

    fhip_tensor4 c4() const {
        static_assert(R == 4, "rank-4 only");
        fhip_tensor4 t{};
        t.ptr = buf_->ptr();
        t.offset = offset_;
        for (int i = 0; i < 4; i++) {
            t.shape[i] = shape_[i];
            t.stride[i] = stride_[i];
        }
        return t;
    }
    fhip_tensor2 c2() const {
        static_assert(R == 2, "rank-2 only");
        fhip_tensor2 t{};
        t.ptr = buf_->ptr();
        t.offset = offset_;
        for (int i = 0; i < 2; i++) {
            t.shape[i] = shape_[i];
            t.stride[i] = stride_[i];
        }
        return t;
    }

    /// fusor::Tensor<4,D>::flash_attention(&self, k, v, scale, mask) -> Self
    /// (fusor flash_attention.rs:52-73).  `analytic` is the extension MaskCache::get_analytic hands
    /// out when it built the mask itself; it replaces the dense mask tensor.
    Tensor flash_attention(const Tensor &k, const Tensor &v, float scale,
                           std::optional<std::pair<const Tensor<2> *, MaskKind>> mask = std::nullopt,
                           const fhip_analytic_mask *analytic = nullptr, const int32_t *kv_lens = nullptr,
                           const void *mask_intervals = nullptr) const {
        static_assert(R == 4, "flash_attention takes rank-4 tensors");
        if (!device().same(k.device()) || !device().same(v.device()))
            throw Panic("Cannot mix tensors of different devices");  // fusor lib.rs:265
        fhip_attn_args a{};
        Tensor out = empty(device(), dtype_, shape_);  // fresh, contiguous, Q's shape (core :505-507)
        a.q = c4();
        a.k = k.c4();
        a.v = v.c4();
        a.out = out.c4();
        a.dtype = a.out_dtype = (fhip_dtype)dtype_;
        a.scale = scale;
        if (mask) {
            if (!device().same(mask->first->device()))
                throw Panic("Mask must be on the same device as other tensors");  // fusor flash_attention.rs:64
            a.mask = mask->first->c2();
            a.mask_kind = (fhip_mask_kind)mask->second;
            a.mask_intervals = mask_intervals;  // AttentionMask::intervals() of this very mask, or nullptr
        }
        if (analytic) a.analytic = *analytic;
        a.kv_lens = kv_lens;
        size_t need = 0;
        check(fhip_flash_attention_workspace_bytes(&a, device().info().compute_units, &need));
        if (need) {
            a.workspace = device().workspace(need);
            a.workspace_bytes = device().workspace_bytes();
        }
        check(fhip_flash_attention(device().stream(), &a));
        return out;
    }

    template <int>
    friend class Tensor;
    friend class KvCache;
};

/// fusor::cache::AttentionMask (attention_mask.rs:9-83)
class AttentionMask {
    Tensor<2> mask_;
    std::optional<fhip_analytic_mask> analytic_;
    std::shared_ptr<Buffer> intervals_;  // the mask's interval table, computed on first use (the mask never changes)

   public:
    AttentionMask() = default;
    explicit AttentionMask(Tensor<2> mask, std::optional<fhip_analytic_mask> analytic = std::nullopt)
        : mask_(std::move(mask)), analytic_(analytic) {}
    /// AttentionMask::causal(device, seq_len): mask[i][j] = -inf if j > i else 0
    static AttentionMask causal(const Device &dev, uint32_t seq_len, DType dt = DType::F32) {
        std::vector<char> host((size_t)seq_len * seq_len * dtype_bytes(dt));
        check(fhip_mask_causal((fhip_dtype)dt, seq_len, host.data()));
        const uint32_t shape[2] = {seq_len, seq_len};
        fhip_analytic_mask am{1, 1, 0, 0};
        return AttentionMask(Tensor<2>::from_slice(dev, dt, shape, host.data()), am);
    }
    const Tensor<2> &mask() const { return mask_; }
    const std::optional<fhip_analytic_mask> &analytic() const { return analytic_; }
    /// The table fhip_mask_intervals computes for this mask, to be passed to flash_attention with it: the calls then
    /// skip their scan of the tensor (one mask serves every layer of a forward pass).
    const void *intervals() {
        if (!intervals_) {
            size_t bytes = 0;
            check(fhip_mask_intervals_bytes(mask_.shape()[0], &bytes));
            intervals_ = std::make_shared<Buffer>(mask_.device(), bytes);
            const fhip_tensor2 view = mask_.c2();
            check(fhip_mask_intervals(mask_.device().stream(), &view, (fhip_dtype)mask_.dtype(), intervals_->ptr(), bytes));
        }
        return intervals_->ptr();
    }
};

/// fusor::cache::MaskCache (mask_cache.rs:9-116): base masks cached by (seq_len, window)
class MaskCache {
    DType dtype_;
    std::map<std::pair<uint32_t, int64_t>, AttentionMask> masks_;

   public:
    explicit MaskCache(DType dt = DType::F32) : dtype_(dt) {}
    /// get_mask(seq_len, seqlen_offset, sliding_window_size, device)
    AttentionMask get_mask(uint32_t seq_len, uint64_t seqlen_offset, std::optional<uint64_t> sliding_window_size,
                           const Device &dev) {
        const int has_w = sliding_window_size.has_value();
        const uint64_t w = has_w ? *sliding_window_size : 0;
        uint32_t rows;
        uint64_t cols;
        check(fhip_mask_get_mask_shape(seq_len, seqlen_offset, has_w, w, &rows, &cols));
        fhip_analytic_mask am{};
        const bool have_am = fhip_mask_get_analytic(seq_len, seqlen_offset, has_w, w, &am) == FHIP_OK;
        const auto key = std::make_pair(seq_len, has_w ? (int64_t)w : (int64_t)-1);
        // the tensors are written by a kernel (bit for bit what the reference's host loops build)
        auto it = masks_.find(key);
        if (it == masks_.end()) {
            const uint32_t shape[2] = {seq_len, seq_len};
            Tensor<2> base = Tensor<2>::empty(dev, dtype_, shape);
            check(fhip_mask_get_mask_device(dev.stream(), (fhip_dtype)dtype_, seq_len, 0, has_w, w, base.c2().ptr));
            it = masks_.emplace(key, AttentionMask(base)).first;
        }
        std::optional<fhip_analytic_mask> oam;
        if (have_am) oam = am;
        if (cols > seq_len) {  // left padding with zeros (mask_cache.rs:73-85)
            const uint32_t shape[2] = {rows, (uint32_t)cols};
            Tensor<2> full = Tensor<2>::empty(dev, dtype_, shape);
            check(fhip_mask_get_mask_device(dev.stream(), (fhip_dtype)dtype_, seq_len, seqlen_offset, has_w, w, full.c2().ptr));
            return AttentionMask(full, oam);
        }
        return AttentionMask(it->second.mask(), oam);
    }
};

/// fusor::cache::KvCache over device memory (kv_cache.rs:13-68, tensor_cache.rs:9-124)
class KvCache {
    struct Inner {
        fhip_kv_cache *c = nullptr;
        ~Inner() {
            if (c) fhip_kv_cache_destroy(c);
        }
    };
    std::shared_ptr<Inner> in_;
    Device dev_;
    DType dtype_;

   public:
    /// KvCache::new(concat_dim, max_sequence_len); the device cache concatenates along dim 2
    KvCache(const Device &dev, int concat_dim, uint64_t max_sequence_len, DType dt = DType::F32)
        : in_(std::make_shared<Inner>()), dev_(dev), dtype_(dt) {
        if (concat_dim != 2) throw GpuError("the device KV cache concatenates [B, Hkv, seq, D] along dim 2");
        check(fhip_kv_cache_create(dev.handle(), (fhip_dtype)dt, max_sequence_len, &in_->c));
    }
    void reset() { check(fhip_kv_cache_reset(in_->c)); }
    uint64_t current_seq_len() const {
        uint64_t n;
        check(fhip_kv_cache_current_seq_len(in_->c, &n));
        return n;
    }
    /// append(device, k, v) -> (keys, values) including the new rows
    std::pair<Tensor<4>, Tensor<4>> append(const Device &, const Tensor<4> &k, const Tensor<4> &v) {
        fhip_tensor4 kn = k.c4(), vn = v.c4(), ka{}, va{};
        check(fhip_kv_cache_append(in_->c, dev_.stream(), &kn, &vn, &ka, &va));
        auto wrap = [&](const fhip_tensor4 &t) {
            Tensor<4> r(std::make_shared<Buffer>(dev_, t.ptr), dtype_, t.shape, t.stride, t.offset, in_);
            return r;
        };
        return {wrap(ka), wrap(va)};
    }
    /// append(rope(k), v): the rotation of RopeCache::forward / forward_interleaved and the conversion to
    /// the cache's element type happen in the pass that writes the new rows
    /// q_out = rope(norm(q)) and append(rope(norm(k)), v) in ONE launch (a decode step's three tiny row-wise jobs);
    /// returns (k_all, v_all); q_out is a pre-allocated tensor of q's shape
    std::pair<Tensor<4>, Tensor<4>> qkv_rope_append(const fhip_rope_tables &tables, const Tensor<4> &q, Tensor<4> &q_out,
                                                    const Tensor<4> &k, const Tensor<4> &v,
                                                    const fhip_rms_norm *q_norm = nullptr, const fhip_rms_norm *k_norm = nullptr) {
        if (k.dtype() != v.dtype()) throw Panic("qkv_rope_append: keys and values differ in element type");
        fhip_tensor4 qn = q.c4(), qo = q_out.c4(), kn = k.c4(), vn = v.c4(), ka{}, va{};
        check(fhip_kv_cache_qkv_rope_append(in_->c, dev_.stream(), q_norm, k_norm, &tables, &qn, (fhip_dtype)q.dtype(), &qo,
                                            (fhip_dtype)q_out.dtype(), &kn, &vn, (fhip_dtype)k.dtype(), &ka, &va));
        auto wrap = [&](const fhip_tensor4 &t) {
            Tensor<4> r(std::make_shared<Buffer>(dev_, t.ptr), dtype_, t.shape, t.stride, t.offset, in_);
            return r;
        };
        return {wrap(ka), wrap(va)};
    }
    /// k_norm (RmsNorm::c()): the keys are RMS-normalised before the rotation (attention_k_norm)
    std::pair<Tensor<4>, Tensor<4>> append_rope(const fhip_rope_tables &tables, const Tensor<4> &k, const Tensor<4> &v,
                                                const fhip_rms_norm *k_norm = nullptr) {
        if (k.dtype() != v.dtype()) throw Panic("append_rope: keys and values differ in element type");
        fhip_tensor4 kn = k.c4(), vn = v.c4(), ka{}, va{};
        if (k_norm)
            check(fhip_kv_cache_norm_rope_append(in_->c, dev_.stream(), k_norm, &tables, &kn, &vn, (fhip_dtype)k.dtype(), &ka, &va));
        else
            check(fhip_kv_cache_rope_append(in_->c, dev_.stream(), &tables, &kn, &vn, (fhip_dtype)k.dtype(), &ka, &va));
        auto wrap = [&](const fhip_tensor4 &t) {
            Tensor<4> r(std::make_shared<Buffer>(dev_, t.ptr), dtype_, t.shape, t.stride, t.offset, in_);
            return r;
        };
        return {wrap(ka), wrap(va)};
    }
};

/// fusor::RopeCache (fusor-ml/fusor/src/composite/rope.rs:180-265): [context_length, head_dim/2] f32
/// cos/sin tables on the device, applied by one fused kernel per tensor.
class RopeCache {
    Tensor<2> cos_, sin_;
    Device dev_;
    uint64_t rows_;

   public:
    /// RopeCache::from_parts(cos, sin): host tables, row-major [rows, head_dim / 2]
    RopeCache(const Device &dev, uint32_t rows, uint32_t half_dim, const float *cos, const float *sin)
        : cos_(Tensor<2>::from_slice(dev, DType::F32, {rows, half_dim}, cos)),
          sin_(Tensor<2>::from_slice(dev, DType::F32, {rows, half_dim}, sin)), dev_(dev), rows_(rows) {}
    /// RopeCache::new(head_dim, context_length, rope_theta, device) (rope.rs:198-221)
    static RopeCache standard(const Device &dev, uint32_t head_dim, uint32_t context_length, float rope_theta) {
        const uint32_t half = head_dim / 2;
        std::vector<float> c((size_t)context_length * half), s(c.size());
        for (uint32_t i = 0; i < half; i++) {
            const float inv = 1.0f / std::pow(rope_theta, (float)(2 * i) / (float)head_dim);  // base_inverse_frequency
            for (uint32_t p = 0; p < context_length; p++) {
                const float a = (float)p * inv;
                c[(size_t)p * half + i] = std::cos(a);
                s[(size_t)p * half + i] = std::sin(a);
            }
        }
        return RopeCache(dev, context_length, half, c.data(), s.data());
    }
    fhip_rope_tables tables(uint64_t start_pos, bool interleaved) const {
        fhip_rope_tables t{};
        t.cos = (const float *)cos_.c2().ptr;
        t.sin = (const float *)sin_.c2().ptr;
        t.table_rows = rows_;
        t.start_pos = start_pos;
        t.interleaved = interleaved ? 1 : 0;
        return t;
    }
    /// norm (RmsNorm::c()): the rows are RMS-normalised first, in the same pass (attention_q_norm)
    Tensor<4> apply(const Tensor<4> &x, uint64_t start_pos, bool interleaved, std::optional<DType> out_dtype = std::nullopt,
                    const fhip_rms_norm *norm = nullptr) const {
        const DType od = out_dtype.value_or(x.dtype());
        const auto &shp = x.shape();
        Tensor<4> out = Tensor<4>::empty(dev_, od, {shp[0], shp[1], shp[2], shp[3]});
        const fhip_rope_tables t = tables(start_pos, interleaved);
        const fhip_tensor4 cx = x.c4(), co = out.c4();
        if (norm)
            check(fhip_norm_rope(dev_.stream(), norm, &t, &cx, (fhip_dtype)x.dtype(), &co, (fhip_dtype)od));
        else
            check(fhip_rope(dev_.stream(), &t, &cx, (fhip_dtype)x.dtype(), &co, (fhip_dtype)od));
        return out;
    }
    /// RopeCache::forward(q, k, start_pos) -> (q, k)   (pairs (i, i + head_dim/2))
    std::pair<Tensor<4>, Tensor<4>> forward(const Tensor<4> &q, const Tensor<4> &k, uint64_t start_pos) const {
        return {apply(q, start_pos, false), apply(k, start_pos, false)};
    }
    /// RopeCache::forward_interleaved(q, k, start_pos) -> (q, k)   (pairs (2i, 2i + 1))
    std::pair<Tensor<4>, Tensor<4>> forward_interleaved(const Tensor<4> &q, const Tensor<4> &k, uint64_t start_pos) const {
        return {apply(q, start_pos, true), apply(k, start_pos, true)};
    }
};

/// fusor::layers::RmsNorm<1, T> over the last dimension (fusor-ml/fusor/src/layers/rms_norm.rs:11-133), as the
/// q / k norm of attention blocks uses it; pass c() to RopeCache::apply / KvCache::append_rope to fuse it.
class RmsNorm {
    Tensor<2> weight_;
    std::optional<Tensor<2>> bias_;
    Device dev_;
    DType dtype_;
    float eps_;

   public:
    /// RmsNorm::new(weight, bias, eps): host values [head_dim] in f32, stored as `dtype`
    RmsNorm(const Device &dev, DType dtype, uint32_t head_dim, const float *weight, const float *bias, float eps)
        : weight_(Tensor<2>::from_slice(dev, dtype, {1, head_dim}, weight)), dev_(dev), dtype_(dtype), eps_(eps) {
        if (bias) bias_ = Tensor<2>::from_slice(dev, dtype, {1, head_dim}, bias);
    }
    float eps() const { return eps_; }
    fhip_rms_norm c() const {
        fhip_rms_norm n{};
        n.weight = weight_.c2().ptr;
        n.bias = bias_ ? bias_->c2().ptr : nullptr;
        n.dtype = (fhip_dtype)dtype_;
        n.eps = eps_;
        return n;
    }
    /// RmsNorm::forward_generic_4d (rms_norm.rs:122-133): the norm alone
    Tensor<4> forward_generic_4d(const Tensor<4> &x) const {
        const auto &shp = x.shape();
        Tensor<4> out = Tensor<4>::empty(dev_, x.dtype(), {shp[0], shp[1], shp[2], shp[3]});
        const fhip_rms_norm n = c();
        const fhip_tensor4 cx = x.c4(), co = out.c4();
        check(fhip_norm_rope(dev_.stream(), &n, nullptr, &cx, (fhip_dtype)x.dtype(), &co, (fhip_dtype)x.dtype()));
        return out;
    }
};

}  // namespace fusor_hip
