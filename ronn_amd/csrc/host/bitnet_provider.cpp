// Implementation of the MI355X BitNet execution provider (host side); see the header.
#include "bitnet_provider.hpp"

#include <cstdio>

#include <chrono>
#include <cstring>
#include <sstream>

namespace ronn {
namespace bitnet {

void check(int rc, const char *what) {
    if (rc != RBN_OK)
        throw Error(std::string(what) + ": " + rbn_last_error() + " (status " + std::to_string(rc) +
                    ")");
}

Device::Device(int index) : index_(index) { check(rbn_ctx_create(index, &ctx_), "rbn_ctx_create"); }
Device::~Device() { rbn_ctx_destroy(ctx_); }

namespace {

// RAII device buffer on a Device.
struct DBuf {
    rbn_ctx *ctx;
    void *p = nullptr;
    DBuf(rbn_ctx *c, size_t bytes) : ctx(c) { check(rbn_malloc(c, bytes, &p), "rbn_malloc"); }
    ~DBuf() {
        if (p) rbn_free(ctx, p);
    }
    DBuf(const DBuf &) = delete;
    DBuf &operator=(const DBuf &) = delete;
    void *release() {
        void *r = p;
        p = nullptr;
        return r;
    }
};

std::string shape_str(const std::vector<size_t> &s) {
    std::ostringstream o;
    o << "[";
    for (size_t i = 0; i < s.size(); ++i) o << (i ? ", " : "") << s[i];
    o << "]";
    return o.str();
}

// Second digest of the same bytes, unrelated to hash_floats (byte-wise FNV-1a folded with the
// position): a cache hit needs both to agree.
uint64_t check_bytes(const void *data, size_t bytes) {
    const uint8_t *p = static_cast<const uint8_t *>(data);
    uint64_t a = 0xcbf29ce484222325ull, b = 0x84222325cbf29ce4ull;
    size_t i = 0;
    for (; i + 8 <= bytes; i += 8) {
        uint64_t x;
        std::memcpy(&x, p + i, 8);
        a = (a ^ x) * 0x100000001b3ull;
        b = (b + x) * 0xff51afd7ed558ccdull + (b >> 31);
    }
    for (; i < bytes; ++i) a = (a ^ p[i]) * 0x100000001b3ull;
    return a ^ (b << 1) ^ bytes;
}

// 64-bit content hash of a weight tensor (four interleaved multiply-xor lanes).
uint64_t hash_floats(const std::vector<float> &v, const std::vector<size_t> &shape) {
    const uint64_t kMul = 0x9E3779B97F4A7C15ull;
    uint64_t h[4] = {0x243F6A8885A308D3ull, 0x13198A2E03707344ull, 0xA4093822299F31D0ull,
                     0x082EFA98EC4E6C89ull};
    const size_t n64 = v.size() / 2;
    const uint64_t *p = reinterpret_cast<const uint64_t *>(v.data());
    size_t i = 0;
    for (; i + 4 <= n64; i += 4) {
        for (int j = 0; j < 4; ++j) {
            uint64_t x;
            std::memcpy(&x, p + i + j, 8);
            h[j] = (h[j] ^ x) * kMul;
            h[j] ^= h[j] >> 29;
        }
    }
    uint64_t r = v.size() * kMul;
    for (; i < n64; ++i) {
        uint64_t x;
        std::memcpy(&x, p + i, 8);
        r = (r ^ x) * kMul;
    }
    if (v.size() & 1) {
        uint32_t x;
        std::memcpy(&x, &v.back(), 4);
        r = (r ^ x) * kMul;
    }
    for (size_t d : shape) r = (r ^ d) * kMul;
    for (int j = 0; j < 4; ++j) r = (r ^ h[j]) * kMul;
    return r ^ (r >> 32);
}

void require_f32(const Tensor &t) {
    if (t.dtype() != DataType::F32)  // quantization.rs:68-72
        throw Error("BitNet quantization requires FP32 input tensors");
}

}  // namespace

// ---- quantization.rs --------------------------------------------------------------------

int8_t TernaryTensor::get_value(size_t index) const {
    if (index >= element_count) return 0;  // :276-278
    const unsigned bit_pair = (packed_data[index / 4] >> ((index % 4) * 2)) & 3u;
    switch (bit_pair) {  // :285-290
        case 0: return -1;
        case 1: return 0;
        case 2: return 1;
        default: return 0;
    }
}

TernaryTensor BitNetQuantizer::quantize_ternary(const Tensor &input) const {
    require_f32(input);
    rbn_ctx *ctx = device_->ctx();
    const std::vector<float> &data = input.to_vec();  // :74
    const size_t n = data.size();
    TernaryTensor t;
    t.shape = input.shape();
    t.element_count = n;
    t.packed_data.assign((n + 3) / 4, 0);
    DBuf d_x(ctx, n * 4), d_p(ctx, rbn_packed_capacity(n));
    check(rbn_h2d(ctx, d_x.p, data.data(), n * 4), "rbn_h2d");
    check(rbn_quantize_ternary(ctx, (const float *)d_x.p, n, sum_mode_, (uint8_t *)d_p.p, &t.scale,
                               &t.threshold, nullptr),
          "rbn_quantize_ternary");
    check(rbn_d2h(ctx, t.packed_data.data(), d_p.p, t.packed_data.size()), "rbn_d2h");
    return t;
}

Tensor BitNetQuantizer::dequantize_ternary(const TernaryTensor &t) const {
    rbn_ctx *ctx = device_->ctx();
    const size_t n = t.element_count;
    DBuf d_p(ctx, rbn_packed_capacity(n)), d_o(ctx, n * 4);
    check(rbn_h2d(ctx, d_p.p, t.packed_data.data(), t.packed_data.size()), "rbn_h2d");
    check(rbn_dequantize_ternary(ctx, (const uint8_t *)d_p.p, n, t.scale, (float *)d_o.p),
          "rbn_dequantize_ternary");
    std::vector<float> out(n);
    check(rbn_d2h(ctx, out.data(), d_o.p, n * 4), "rbn_d2h");
    return Tensor::from_data(std::move(out), t.shape, DataType::F32, TensorLayout::RowMajor);
}

// ---- kernels.rs ----------------------------------------------------------------------------

BitNetKernel::BitNetKernel(BitNetOperation operation, QuantizationMethod method,
                           std::shared_ptr<Device> device, ActivationMode act_mode, int sum_mode,
                           bool cache_weights, size_t max_cache_bytes)
    : operation_(operation),
      method_(method),
      device_(std::move(device)),
      act_mode_(act_mode),
      sum_mode_(sum_mode),
      cache_weights_(cache_weights),
      max_cache_bytes_(max_cache_bytes) {}

BitNetKernel::~BitNetKernel() {
    for (auto &kv : weight_cache_) rbn_free(device_->ctx(), kv.second.d_tiled);
}

void BitNetKernel::update_stats(double us) {  // kernels.rs:235-251
    stats_.execution_count += 1;
    if (stats_.execution_count == 1) {
        stats_.min_time_us = stats_.max_time_us = stats_.average_time_us = us;
    } else {
        if (us < stats_.min_time_us) stats_.min_time_us = us;
        if (us > stats_.max_time_us) stats_.max_time_us = us;
        const double n = (double)stats_.execution_count;
        stats_.average_time_us = ((n - 1.0) * stats_.average_time_us + us) / n;
    }
}

Tensor BitNetKernel::execute_ternary_matmul(const Tensor &a, const Tensor &b) {
    require_f32(a);
    require_f32(b);
    // Dimensions: explicit ones are checked as in kernels.rs:142-152; 0,0,0 infers them.
    size_t m = operation_.m, n = operation_.n, k = operation_.k;
    const bool infer = (m == 0 && n == 0 && k == 0);
    if (infer) {
        if (a.shape().size() != 2 || b.shape().size() != 2 || a.shape()[1] != b.shape()[0])
            throw Error("Matrix dimension mismatch: A=" + shape_str(a.shape()) +
                        ", B=" + shape_str(b.shape()) + ", expected A=[m,k], B=[k,n]");
        m = a.shape()[0];
        k = a.shape()[1];
        n = b.shape()[1];
    }
    if (a.shape() != std::vector<size_t>{m, k} || b.shape() != std::vector<size_t>{k, n}) {
        std::ostringstream o;
        o << "Matrix dimension mismatch: A=" << shape_str(a.shape()) << ", B=" << shape_str(b.shape())
          << ", expected A=[" << m << "," << k << "], B=[" << k << "," << n << "]";
        throw Error(o.str());
    }
    if (m == 0 || n == 0 || k == 0)
        return Tensor::from_data(std::vector<float>(m * n, 0.0f), {m, n}, DataType::F32,
                                 TensorLayout::RowMajor);
    // weights: ternarise + tile once per distinct content (kernels.rs:278 does it per call)
    bool owned = false;
    const std::vector<float> bv = b.to_vec();
    const uint64_t key = cache_weights_ ? hash_floats(bv, b.shape()) : 0;
    const uint64_t chk = cache_weights_ ? check_bytes(bv.data(), bv.size() * 4) : 0;
    CachedWeights w = tiled_weights(key, chk, bv.size() * 4, k, n, nullptr, bv.data(), 1.0f, &owned);
    struct Release {
        rbn_ctx *c;
        void *p;
        ~Release() {
            if (p) rbn_free(c, p);
        }
    } release{device_->ctx(), owned ? w.d_tiled : nullptr};
    return multiply(a, m, k, n, w.d_tiled, w.scale);
}

BitNetKernel::CachedWeights BitNetKernel::tiled_weights(uint64_t key, uint64_t check_digest,
                                                        size_t source_bytes, size_t k, size_t n,
                                                        const uint8_t *h_packed, const float *h_f32,
                                                        float scale, bool *owned) {
    rbn_ctx *ctx = device_->ctx();
    CachedWeights w;
    *owned = false;
    if (cache_weights_) {
        auto it = weight_cache_.find(key);
        if (it != weight_cache_.end()) {
            CachedWeights &c = it->second;
            // the key alone is not trusted: a collision would multiply with another matrix
            if (c.k == k && c.n == n && c.source_bytes == source_bytes && c.check == check_digest) {
                c.last_use = ++use_clock_;
                return c;
            }
            check(rbn_free(ctx, c.d_tiled), "rbn_free");
            cache_bytes_ -= c.bytes;
            weight_cache_.erase(it);
        }
    }
    DBuf d_p(ctx, rbn_packed_capacity(k * n));
    DBuf d_t(ctx, rbn_tiled_bytes(k, n));
    if (h_f32) {
        DBuf d_b(ctx, k * n * 4);
        float thr = 0.0f;
        check(rbn_h2d(ctx, d_b.p, h_f32, k * n * 4), "rbn_h2d");
        check(rbn_quantize_ternary(ctx, (const float *)d_b.p, k * n, sum_mode_, (uint8_t *)d_p.p,
                                   &w.scale, &thr, nullptr),
              "rbn_quantize_ternary");
    } else {
        check(rbn_fill_u8(ctx, d_p.p, 0x55, rbn_packed_capacity(k * n)), "rbn_fill_u8");  // code 01 = 0
        check(rbn_h2d(ctx, d_p.p, h_packed, (k * n + 3) / 4), "rbn_h2d");
        w.scale = scale;
    }
    check(rbn_tile_weights(ctx, (const uint8_t *)d_p.p, k, n, (uint32_t *)d_t.p), "rbn_tile_weights");
    check(rbn_sync(ctx), "rbn_sync");
    w.bytes = rbn_tiled_bytes(k, n);
    w.d_tiled = d_t.release();
    w.k = k;
    w.n = n;
    w.source_bytes = source_bytes;
    w.check = check_digest;
    w.last_use = ++use_clock_;
    // make room: the least recently used matrices go first (every caller holds the kernel's
    // lock for the whole call, so nothing evicted here is in use)
    while (cache_weights_ && w.bytes <= max_cache_bytes_ && cache_bytes_ + w.bytes > max_cache_bytes_ &&
           !weight_cache_.empty()) {
        auto oldest = weight_cache_.end();
        for (auto it = weight_cache_.begin(); it != weight_cache_.end(); ++it)
            if (!pinned_.count(it->first) &&
                (oldest == weight_cache_.end() || it->second.last_use < oldest->second.last_use))
                oldest = it;
        if (oldest == weight_cache_.end()) break;  // everything left is in use by this call
        check(rbn_free(ctx, oldest->second.d_tiled), "rbn_free");
        cache_bytes_ -= oldest->second.bytes;
        weight_cache_.erase(oldest);
    }
    if (cache_weights_ && cache_bytes_ + w.bytes <= max_cache_bytes_) {
        weight_cache_[key] = w;
        cache_bytes_ += w.bytes;
        memory_usage_.current_bytes = cache_bytes_;
        if (cache_bytes_ > memory_usage_.peak_bytes) memory_usage_.peak_bytes = cache_bytes_;
        memory_usage_.allocation_count += 1;
    } else {
        *owned = true;
    }
    return w;
}

Tensor BitNetKernel::multiply(const Tensor &a, size_t m, size_t k, size_t n, const void *d_tiled,
                              float w_scale) {
    rbn_ctx *ctx = device_->ctx();
    // activations (kernels.rs:277): per-tensor ternary as the reference, or per-token int8
    DBuf d_a(ctx, m * k * 4), d_q(ctx, m * rbn_act_pitch(k)), d_s(ctx, m * 4), d_r(ctx, m * 4);
    DBuf d_o(ctx, m * n * 4);
    check(rbn_h2d(ctx, d_a.p, a.to_vec().data(), m * k * 4), "rbn_h2d");
    if (act_mode_ == ActivationMode::Ternary) {
        check(rbn_act_quant_ternary(ctx, (const float *)d_a.p, m, k, sum_mode_, (int8_t *)d_q.p,
                                    (float *)d_s.p, (int32_t *)d_r.p, nullptr, nullptr),
              "rbn_act_quant_ternary");
    } else {
        check(rbn_act_quant_i8(ctx, (const float *)d_a.p, m, k, (int8_t *)d_q.p, (float *)d_s.p,
                               (int32_t *)d_r.p),
              "rbn_act_quant_i8");
    }
    // kernels.rs:280-281 and the epilogue of :168
    check(rbn_matmul_t2_i8(ctx, (const int8_t *)d_q.p, (const float *)d_s.p, (const int32_t *)d_r.p,
                           (const uint32_t *)d_tiled, w_scale, m, k, n, nullptr, (float *)d_o.p),
          "rbn_matmul_t2_i8");
    std::vector<float> result(m * n);
    check(rbn_d2h(ctx, result.data(), d_o.p, m * n * 4), "rbn_d2h");
    return Tensor::from_data(std::move(result), {m, n}, DataType::F32, TensorLayout::RowMajor);
}

std::vector<Tensor> BitNetKernel::execute_group(const std::vector<Tensor> &inputs, int *launches) {
    const auto start = std::chrono::steady_clock::now();
    std::lock_guard<std::mutex> guard(lock_);
    if (launches) *launches = 0;
    if (operation_.kind != BitNetOperation::TernaryMatMul)
        throw Error("execute_group needs a TernaryMatMul kernel");
    if (inputs.empty() || inputs.size() % 2 != 0)
        throw Error("Ternary MatMul group requires pairs of inputs (A_i, B_i)");
    const size_t count = inputs.size() / 2;
    // every node is checked as execute() checks it (kernels.rs:142-152, quantization.rs:68-72)
    const Tensor &a0 = inputs[0], &b0 = inputs[1];
    for (const Tensor &t : inputs) require_f32(t);
    if (a0.shape().size() != 2 || b0.shape().size() != 2 || a0.shape()[1] != b0.shape()[0])
        throw Error("Matrix dimension mismatch: A=" + shape_str(a0.shape()) + ", B=" + shape_str(b0.shape()) +
                    ", expected A=[m,k], B=[k,n]");
    const size_t m = a0.shape()[0], k = a0.shape()[1], n = b0.shape()[1];
    if ((operation_.m || operation_.n || operation_.k) &&
        (operation_.m != m || operation_.n != n || operation_.k != k)) {
        std::ostringstream o;
        o << "Matrix dimension mismatch: A=" << shape_str(a0.shape()) << ", B=" << shape_str(b0.shape())
          << ", expected A=[" << operation_.m << "," << operation_.k << "], B=[" << operation_.k << ","
          << operation_.n << "]";
        throw Error(o.str());
    }
    for (size_t i = 1; i < count; ++i)
        if (inputs[2 * i].shape() != a0.shape() || inputs[2 * i + 1].shape() != b0.shape())
            throw Error("Ternary MatMul group: node " + std::to_string(i) + " has A=" +
                        shape_str(inputs[2 * i].shape()) + ", B=" + shape_str(inputs[2 * i + 1].shape()) +
                        ", the group's shape is A=" + shape_str(a0.shape()) + ", B=" + shape_str(b0.shape()));
    std::vector<Tensor> results;
    if (m == 0 || n == 0 || k == 0) {
        for (size_t i = 0; i < count; ++i)
            results.push_back(Tensor::from_data(std::vector<float>(m * n, 0.0f), {m, n}, DataType::F32,
                                                TensorLayout::RowMajor));
        return results;
    }
    rbn_ctx *ctx = device_->ctx();
    // weights: ternarised and tiled once per distinct matrix, as in execute(); cached ones are
    // pinned for the duration of the call, the others are freed at its end
    struct Held {
        rbn_ctx *c;
        std::vector<void *> owned;
        std::set<uint64_t> *pins;
        ~Held() {
            for (void *p : owned) rbn_free(c, p);
            pins->clear();
        }
    } held{ctx, {}, &pinned_};
    std::vector<CachedWeights> w(count);
    for (size_t i = 0; i < count; ++i) {
        const Tensor &b = inputs[2 * i + 1];
        const std::vector<float> &bv = b.to_vec();
        const uint64_t key = cache_weights_ ? hash_floats(bv, b.shape()) : 0;
        const uint64_t chk = cache_weights_ ? check_bytes(bv.data(), bv.size() * 4) : 0;
        bool owned = false;
        w[i] = tiled_weights(key, chk, bv.size() * 4, k, n, nullptr, bv.data(), 1.0f, &owned);
        if (owned)
            held.owned.push_back(w[i].d_tiled);
        else
            pinned_.insert(key);
    }
    // activations: nodes that share their input (q/k/v, gate/up) are quantised once
    struct Acts {
        std::unique_ptr<DBuf> q, s, r;
    };
    std::vector<Acts> acts;
    std::vector<size_t> acts_of(count), first_with(0);
    for (size_t i = 0; i < count; ++i) {
        const std::vector<float> &av = inputs[2 * i].to_vec();
        size_t j = 0;
        for (; j < first_with.size(); ++j) {
            const std::vector<float> &other = inputs[2 * first_with[j]].to_vec();
            if (&other == &av || std::memcmp(other.data(), av.data(), av.size() * 4) == 0) break;
        }
        acts_of[i] = j;
        if (j < first_with.size()) continue;
        first_with.push_back(i);
        DBuf d_a(ctx, m * k * 4);
        Acts x;
        x.q.reset(new DBuf(ctx, m * rbn_act_pitch(k)));
        x.s.reset(new DBuf(ctx, m * 4));
        x.r.reset(new DBuf(ctx, m * 4));
        check(rbn_h2d(ctx, d_a.p, av.data(), m * k * 4), "rbn_h2d");
        if (act_mode_ == ActivationMode::Ternary)
            check(rbn_act_quant_ternary(ctx, (const float *)d_a.p, m, k, sum_mode_, (int8_t *)x.q->p,
                                        (float *)x.s->p, (int32_t *)x.r->p, nullptr, nullptr),
                  "rbn_act_quant_ternary");
        else
            check(rbn_act_quant_i8(ctx, (const float *)d_a.p, m, k, (int8_t *)x.q->p, (float *)x.s->p,
                                   (int32_t *)x.r->p),
                  "rbn_act_quant_i8");
        acts.push_back(std::move(x));
    }
    // one output slab, each node's [m,n] block at a 16-byte aligned offset
    const size_t stride = (m * n * 4 + 15) / 16 * 16;
    DBuf d_o(ctx, stride * count);
    const bool decode = m <= RBN_GEMV_MAX_M && rbn_matmul_kernel_choice(m, k, n) == RBN_KERNEL_GEMV;
    int issued = 0;
    if (decode) {
        for (size_t lo = 0; lo < count; lo += RBN_GEMV_GROUP_MAX) {
            const size_t cnt = std::min<size_t>(RBN_GEMV_GROUP_MAX, count - lo);
            std::vector<rbn_gemv_problem> problems(cnt);
            for (size_t i = 0; i < cnt; ++i) {
                const Acts &x = acts[acts_of[lo + i]];
                problems[i].d_q = (const int8_t *)x.q->p;
                problems[i].d_act_scale = (const float *)x.s->p;
                problems[i].d_rowsum = (const int32_t *)x.r->p;
                problems[i].d_tiled = (const uint32_t *)w[lo + i].d_tiled;
                problems[i].w_scale = w[lo + i].scale;
                problems[i].d_acc = nullptr;
                problems[i].d_out = (float *)((char *)d_o.p + (lo + i) * stride);
            }
            check(rbn_gemv_t2_i8_grouped(ctx, problems.data(), cnt, m, k, n), "rbn_gemv_t2_i8_grouped");
            ++issued;
        }
    } else {
        for (size_t i = 0; i < count; ++i) {
            const Acts &x = acts[acts_of[i]];
            check(rbn_matmul_t2_i8(ctx, (const int8_t *)x.q->p, (const float *)x.s->p, (const int32_t *)x.r->p,
                                   (const uint32_t *)w[i].d_tiled, w[i].scale, m, k, n, nullptr,
                                   (float *)((char *)d_o.p + i * stride)),
                  "rbn_matmul_t2_i8");
            ++issued;
        }
    }
    std::vector<uint8_t> slab(stride * count);
    check(rbn_d2h(ctx, slab.data(), d_o.p, slab.size()), "rbn_d2h");
    for (size_t i = 0; i < count; ++i) {
        std::vector<float> r(m * n);
        std::memcpy(r.data(), slab.data() + i * stride, m * n * 4);
        results.push_back(Tensor::from_data(std::move(r), {m, n}, DataType::F32, TensorLayout::RowMajor));
    }
    if (launches) *launches = issued;
    const double us =
        std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - start).count();
    for (size_t i = 0; i < count; ++i) update_stats(us / (double)count);  // one execution per node
    return results;
}

Tensor BitNetKernel::execute_prepacked(const Tensor &a, const TernaryTensor &w) {
    const auto start = std::chrono::steady_clock::now();
    std::lock_guard<std::mutex> guard(lock_);
    if (operation_.kind != BitNetOperation::TernaryMatMul)
        throw Error("execute_prepacked needs a TernaryMatMul kernel");
    require_f32(a);
    validate_ternary_tensor(w);
    if (a.shape().size() != 2 || w.shape.size() != 2 || a.shape()[1] != w.shape[0])
        throw Error("Matrix dimension mismatch: A=" + shape_str(a.shape()) + ", B=" + shape_str(w.shape) +
                    ", expected A=[m,k], B=[k,n]");
    const size_t m = a.shape()[0], k = a.shape()[1], n = w.shape[1];
    if ((operation_.m || operation_.n || operation_.k) &&
        (operation_.m != m || operation_.n != n || operation_.k != k))
        throw Error("Matrix dimension mismatch: the kernel was compiled for other dimensions");
    if (m == 0 || n == 0 || k == 0)
        return Tensor::from_data(std::vector<float>(m * n, 0.0f), {m, n}, DataType::F32,
                                 TensorLayout::RowMajor);
    // cache key: content of the packed bytes, shape and scale
    uint64_t key = 0, chk = 0;
    if (cache_weights_) {
        std::vector<float> as_f((w.packed_data.size() + 3) / 4 + 1, 0.0f);
        std::memcpy(as_f.data(), w.packed_data.data(), w.packed_data.size());
        std::memcpy(&as_f.back(), &w.scale, 4);
        key = hash_floats(as_f, w.shape) ^ 0x5bd1e9955bd1e995ull;
        chk = check_bytes(as_f.data(), as_f.size() * 4);
    }
    bool owned = false;
    CachedWeights cw = tiled_weights(key, chk, w.packed_data.size(), k, n, w.packed_data.data(), nullptr, w.scale,
                                     &owned);
    struct Release {
        rbn_ctx *c;
        void *p;
        ~Release() {
            if (p) rbn_free(c, p);
        }
    } release{device_->ctx(), owned ? cw.d_tiled : nullptr};
    Tensor out = multiply(a, m, k, n, cw.d_tiled, cw.scale);
    update_stats(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - start).count());
    return out;
}

// ---- packed-weight file ----------------------------------------------------------------------
namespace {
uint32_t crc32_ieee(const uint8_t *p, size_t n, uint32_t crc = 0) {
    static uint32_t table[256];
    static bool ready = false;
    if (!ready) {
        for (uint32_t i = 0; i < 256; ++i) {
            uint32_t c = i;
            for (int j = 0; j < 8; ++j) c = (c & 1) ? 0xEDB88320u ^ (c >> 1) : c >> 1;
            table[i] = c;
        }
        ready = true;
    }
    crc = ~crc;
    for (size_t i = 0; i < n; ++i) crc = table[(crc ^ p[i]) & 0xff] ^ (crc >> 8);
    return ~crc;
}
template <typename T>
void put(std::vector<uint8_t> &out, T v) {
    uint8_t b[sizeof(T)];
    std::memcpy(b, &v, sizeof(T));  // the build targets little-endian hosts only
    out.insert(out.end(), b, b + sizeof(T));
}
template <typename T>
T get(const std::vector<uint8_t> &in, size_t &off) {
    if (off + sizeof(T) > in.size()) throw Error("packed-weight file is truncated");
    T v;
    std::memcpy(&v, in.data() + off, sizeof(T));
    off += sizeof(T);
    return v;
}
const char kMagic[8] = {'R', 'B', 'N', 'T', 'E', 'R', 'N', '1'};
}  // namespace

void validate_ternary_tensor(const TernaryTensor &t) {
    size_t n = 1;
    for (size_t d : t.shape) n *= d;
    if (t.shape.empty()) n = t.element_count;
    if (n != t.element_count) throw Error("ternary tensor: shape does not match element_count");
    if (t.packed_data.size() != (t.element_count + 3) / 4)
        throw Error("ternary tensor: packed size is not ceil(element_count / 4)");
    if (t.element_count % 4 != 0 && !t.packed_data.empty()) {
        const unsigned used = (unsigned)(t.element_count % 4) * 2;
        if (t.packed_data.back() >> used) throw Error("ternary tensor: tail bits are not zero");
    }
}

void save_ternary_tensor(const TernaryTensor &t, const std::string &path) {
    validate_ternary_tensor(t);
    if (t.shape.size() > 8) throw Error("ternary tensor: more than 8 dimensions");
    std::vector<uint8_t> out;
    out.reserve(64 + t.packed_data.size());
    out.insert(out.end(), kMagic, kMagic + 8);
    put<uint32_t>(out, 1);
    put<uint32_t>(out, (uint32_t)t.shape.size());
    put<uint64_t>(out, (uint64_t)t.element_count);
    put<float>(out, t.scale);
    put<float>(out, t.threshold);
    put<uint64_t>(out, (uint64_t)t.packed_data.size());
    for (size_t d : t.shape) put<uint64_t>(out, (uint64_t)d);
    out.insert(out.end(), t.packed_data.begin(), t.packed_data.end());
    put<uint32_t>(out, crc32_ieee(out.data(), out.size()));
    FILE *f = std::fopen(path.c_str(), "wb");
    if (!f) throw Error("cannot open " + path + " for writing");
    const size_t w = std::fwrite(out.data(), 1, out.size(), f);
    const int rc = std::fclose(f);
    if (w != out.size() || rc != 0) throw Error("short write to " + path);
}

TernaryTensor load_ternary_tensor(const std::string &path) {
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) throw Error("cannot open " + path);
    std::vector<uint8_t> in;
    uint8_t buf[1 << 16];
    size_t r;
    while ((r = std::fread(buf, 1, sizeof(buf), f)) > 0) in.insert(in.end(), buf, buf + r);
    std::fclose(f);
    if (in.size() < 44 || std::memcmp(in.data(), kMagic, 8) != 0)
        throw Error(path + " is not a packed-weight file");
    size_t off = 8;
    const uint32_t version = get<uint32_t>(in, off), ndim = get<uint32_t>(in, off);
    if (version != 1) throw Error("packed-weight file: unsupported version");
    if (ndim > 8) throw Error("packed-weight file: more than 8 dimensions");
    TernaryTensor t;
    t.element_count = (size_t)get<uint64_t>(in, off);
    t.scale = get<float>(in, off);
    t.threshold = get<float>(in, off);
    const uint64_t packed = get<uint64_t>(in, off);
    for (uint32_t i = 0; i < ndim; ++i) t.shape.push_back((size_t)get<uint64_t>(in, off));
    if (packed > in.size() || off + packed + 4 != in.size())
        throw Error("packed-weight file: size does not match its header");
    t.packed_data.assign(in.begin() + off, in.begin() + off + packed);
    off += packed;
    const uint32_t want = get<uint32_t>(in, off);
    if (crc32_ieee(in.data(), in.size() - 4) != want) throw Error("packed-weight file: checksum mismatch");
    validate_ternary_tensor(t);
    return t;
}

std::vector<Tensor> BitNetKernel::execute(const std::vector<Tensor> &inputs) {
    const auto start = std::chrono::steady_clock::now();
    std::lock_guard<std::mutex> guard(lock_);
    std::vector<Tensor> results;
    switch (operation_.kind) {
        case BitNetOperation::TernaryMatMul:
            if (inputs.size() != 2)  // kernels.rs:272-274
                throw Error("Ternary MatMul requires exactly 2 inputs");
            results.push_back(execute_ternary_matmul(inputs[0], inputs[1]));
            break;
        case BitNetOperation::BinaryMatMul:
            if (inputs.size() != 2) throw Error("Binary MatMul requires exactly 2 inputs");
            throw Error("Binary (XNOR) MatMul is outside this build: it implements the ternary path");
        case BitNetOperation::BinaryElementWise:
            if (inputs.size() != 2)
                throw Error("Binary element-wise operations require exactly 2 inputs");
            throw Error("Binary element-wise kernels are outside this build");
        case BitNetOperation::QuantizedBatchNorm:
            if (inputs.size() < 3) throw Error("Quantized BatchNorm requires at least 3 inputs");
            throw Error("Quantized BatchNorm is outside this build");
    }
    const double us =
        std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - start).count();
    update_stats(us);
    return results;
}

MemoryUsage BitNetKernel::get_memory_usage() const {
    std::lock_guard<std::mutex> guard(lock_);
    return memory_usage_;
}

KernelStats BitNetKernel::get_performance_stats() const {
    std::lock_guard<std::mutex> guard(lock_);
    return stats_;
}

std::unique_ptr<BitNetKernel> create_ternary_matmul_kernel(size_t m, size_t n, size_t k,
                                                           std::shared_ptr<Device> device) {
    BitNetOperation op{BitNetOperation::TernaryMatMul, m, n, k};
    QuantizationMethod method;
    method.kind = QuantizationMethod::Ternary;
    return std::unique_ptr<BitNetKernel>(new BitNetKernel(op, method, std::move(device),
                                                          ActivationMode::Ternary,
                                                          RBN_SUM_STRICT_SEQ, true, 64u << 20));
}

// ---- allocator.rs ----------------------------------------------------------------------------

BitNetMemoryAllocator::BitNetMemoryAllocator(std::shared_ptr<Device> device)
    : device_(std::move(device)) {
    rbn_device_info info;
    check(rbn_get_device_info(device_->ctx(), &info), "rbn_get_device_info");
    total_bytes_ = (size_t)info.hbm_bytes;
}

TensorBuffer BitNetMemoryAllocator::allocate(const std::vector<size_t> &shape, DataType dtype) {
    uint64_t count = 1;
    for (size_t d : shape) count *= d;
    const int64_t size = rbn_tensor_bytes(count, (int)dtype);  // allocator.rs:39-65
    if (size < 0)
        throw Error("Unsupported data type for BitNet allocator: " + std::to_string((int)dtype));
    void *p = nullptr;
    if (rbn_malloc(device_->ctx(), (size_t)size, &p) != RBN_OK)
        throw Error("Memory allocation failed for " + std::to_string(size) + " bytes");
    const size_t now = allocated_.fetch_add((size_t)size) + (size_t)size;  // allocator.rs:78-90
    size_t peak = peak_.load();
    while (now > peak && !peak_.compare_exchange_weak(peak, now)) {
    }
    TensorBuffer b;
    b.ptr = (uint8_t *)p;
    b.size = (size_t)size;
    b.alignment = rbn_tensor_alignment((int)dtype);  // allocator.rs:68-75
    b.memory_type = MemoryType::DeviceMemory;
    return b;
}

void BitNetMemoryAllocator::deallocate(const TensorBuffer &buffer) {
    check(rbn_free(device_->ctx(), buffer.ptr), "rbn_free");
    allocated_.fetch_sub(buffer.size);
}

MemoryInfo BitNetMemoryAllocator::get_memory_info() const {
    MemoryInfo i;
    i.total_bytes = total_bytes_;
    i.allocated_bytes = allocated_.load();
    i.peak_bytes = peak_.load();
    return i;
}

static void recalc(BitNetMemoryStats &s) {  // allocator.rs:194-204
    const size_t total = s.binary_tensor_count + s.ternary_tensor_count;
    if (total > 0)
        s.average_compression_ratio =
            ((float)s.binary_tensor_count * 32.0f + (float)s.ternary_tensor_count * 16.0f) /
            (float)total;
}
void BitNetMemoryStats::add_binary_tensor(size_t original, size_t compressed) {
    binary_tensor_count += 1;
    memory_saved_bytes += original > compressed ? original - compressed : 0;
    recalc(*this);
}
void BitNetMemoryStats::add_ternary_tensor(size_t original, size_t compressed) {
    ternary_tensor_count += 1;
    memory_saved_bytes += original > compressed ? original - compressed : 0;
    recalc(*this);
}

// ---- provider.rs -------------------------------------------------------------------------------

BitNetExecutionProvider::BitNetExecutionProvider(const BitNetProviderConfig &config)
    : config_(config), device_(std::make_shared<Device>(config.device)) {
    allocator_ = std::make_shared<BitNetMemoryAllocator>(device_);
    for (const char *op : {"MatMul", "Gemm", "Conv", "Add", "Sub", "Mul", "And", "Or", "Xor",
                           "BatchNormalization", "ReLU", "Sigmoid"})  // provider.rs:87-99
        supported_ops_.insert(op);
}

bool BitNetExecutionProvider::supports_operation(const std::string &op_type) const {
    return supported_ops_.count(op_type) != 0;
}

float BitNetExecutionProvider::estimate_speedup(const OperatorSpec &op) const {  // :132-150
    const QuantizationMethod::Kind q = config_.quantization_method.kind;
    const std::string &t = op.op_type;
    if (t == "MatMul" || t == "Gemm")
        return q == QuantizationMethod::Binary ? 64.0f : q == QuantizationMethod::Ternary ? 32.0f : 48.0f;
    if (t == "Conv")
        return q == QuantizationMethod::Binary ? 32.0f : q == QuantizationMethod::Ternary ? 24.0f : 28.0f;
    if (t == "Add" || t == "Sub" || t == "Mul") return 16.0f;
    if (t == "And" || t == "Or" || t == "Xor") return 128.0f;
    return 4.0f;
}

ProviderId BitNetExecutionProvider::provider_id() const {
    ProviderId id;
    id.kind = ProviderId::BitNet;
    return id;
}

ProviderCapability BitNetExecutionProvider::get_capability() const {  // :250-271
    ProviderCapability c;
    c.supported_ops = supported_ops_;
    c.data_types = {DataType::Bool, DataType::U8, DataType::F32, DataType::F16};
    c.memory_types = {MemoryType::DeviceMemory};  // the reference reports SystemRAM (:259)
    c.performance_profile = PerformanceProfile::MemoryOptimized;
    c.resource_requirements.has_min_memory = true;
    c.resource_requirements.min_memory_bytes = 16u * 1024 * 1024;
    c.resource_requirements.has_gpu_memory = true;
    c.resource_requirements.gpu_memory_bytes = 16u * 1024 * 1024;
    return c;
}

std::vector<bool> BitNetExecutionProvider::can_handle(const std::vector<OperatorSpec> &ops) const {
    std::vector<bool> r;
    for (const OperatorSpec &op : ops) r.push_back(supports_operation(op.op_type));
    return r;
}

std::unique_ptr<CompiledKernel> BitNetExecutionProvider::create_kernel_for_operation(
    const GraphNode &node) const {
    const std::string &op = node.op_type;
    if (op == "MatMul" || op == "Gemm") {
        if (config_.quantization_method.kind != QuantizationMethod::Ternary)
            throw Error("Binary quantization is outside this build: set quantization_method=ternary");
        // m, n, k come from the inputs at execute() (provider.rs:157-159 hard-codes 64)
        BitNetOperation operation{BitNetOperation::TernaryMatMul, 0, 0, 0};
        return std::unique_ptr<CompiledKernel>(new BitNetKernel(
            operation, config_.quantization_method, device_, config_.activation,
            config_.strict_reference_sum ? RBN_SUM_STRICT_SEQ : RBN_SUM_TREE,
            config_.enable_kernel_caching, config_.max_cache_size));
    }
    if (supported_ops_.count(op))
        throw Error("Operation " + op + " is advertised by the BitNet provider but is outside this "
                    "build, which implements MatMul/Gemm on the ternary path");
    throw Error("Unsupported operation for BitNet: " + op);  // provider.rs:205-208
}

std::unique_ptr<CompiledKernel> BitNetExecutionProvider::compile_subgraph(const SubGraph &subgraph) {
    if (subgraph.nodes.size() != 1)  // provider.rs:297-301
        throw Error("BitNet provider currently supports only single-node subgraphs");
    return create_kernel_for_operation(subgraph.nodes[0]);
}

std::shared_ptr<TensorAllocator> BitNetExecutionProvider::get_allocator() const { return allocator_; }

void BitNetExecutionProvider::configure(const ProviderConfig &config) {  // provider.rs:316-364
    if (config.has_memory_limit) {
        const size_t quarter = config.memory_limit / 4, cap = 128u * 1024 * 1024;
        config_.max_cache_size = quarter < cap ? quarter : cap;
    }
    auto parse_bool = [](const std::string &v, bool dflt) {
        if (v == "true") return true;
        if (v == "false") return false;
        return dflt;
    };
    auto apply_options = [&]() {
        for (const auto &kv : config.custom_options) {
            if (kv.first == "quantization_method") {
                config_.quantization_method.kind =
                    kv.second == "ternary" ? QuantizationMethod::Ternary : QuantizationMethod::Binary;
            } else if (kv.first == "enable_mixed_precision") {
                config_.enable_mixed_precision = parse_bool(kv.second, true);
            } else if (kv.first == "enable_simd") {
                config_.enable_simd = parse_bool(kv.second, true);
            } else if (kv.first == "activation") {
                config_.activation = kv.second == "int8" ? ActivationMode::Int8 : ActivationMode::Ternary;
            } else if (kv.first == "strict_reference_sum") {
                config_.strict_reference_sum = parse_bool(kv.second, true);
            }
        }
    };
    switch (config.optimization_level) {
        case OptimizationLevel::None:
            config_.memory_optimization_level = 0;
            config_.enable_simd = false;
            break;
        case OptimizationLevel::Basic:
            config_.memory_optimization_level = 1;
            config_.enable_simd = true;
            break;
        case OptimizationLevel::Aggressive:
            config_.memory_optimization_level = 2;
            config_.enable_simd = true;
            config_.enable_mixed_precision = true;
            break;
        case OptimizationLevel::Custom: break;
    }
    // The reference parses custom_options only under OptimizationLevel::Custom
    // (provider.rs:336-356), yet its own test expects them to apply under Aggressive
    // (provider.rs:479-500); applying them at every level satisfies both.
    apply_options();
}

void BitNetExecutionProvider::shutdown() { check(rbn_sync(device_->ctx()), "rbn_sync"); }

std::shared_ptr<ExecutionProvider> create_bitnet_provider() {
    return std::make_shared<BitNetExecutionProvider>();
}

std::shared_ptr<ExecutionProvider> create_bitnet_provider_with_config(
    const BitNetProviderConfig &config) {
    return std::make_shared<BitNetExecutionProvider>(config);
}

}  // namespace bitnet
}  // namespace ronn
