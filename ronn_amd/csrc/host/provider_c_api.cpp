// C ABI over the provider mirror (include/ronn_bitnet_provider.h).
#include <string>

#include "../../../include/ronn_bitnet_provider.h"
#include "bitnet_provider.hpp"

using namespace ronn;
using namespace ronn::bitnet;

struct rbp_provider {
    std::shared_ptr<BitNetExecutionProvider> p;
    std::unique_ptr<BitNetQuantizer> quantizer;
};
struct rbp_kernel {
    std::unique_ptr<CompiledKernel> k;
};
struct rbp_ternary {
    TernaryTensor t;
};

namespace {
thread_local std::string g_err;

template <typename F>
int guarded(F &&f) {
    try {
        g_err.clear();
        f();
        return RBP_OK;
    } catch (const std::exception &e) {
        g_err = e.what();
        return RBP_ERR;
    } catch (...) {
        g_err = "unknown error";
        return RBP_ERR;
    }
}

BitNetProviderConfig to_cpp(const rbp_config &c) {
    BitNetProviderConfig o;
    o.quantization_method.kind = c.quantization_method == 0   ? QuantizationMethod::Binary
                                 : c.quantization_method == 1 ? QuantizationMethod::Ternary
                                                              : QuantizationMethod::AsymmetricBinary;
    o.enable_kernel_caching = c.enable_kernel_caching != 0;
    o.max_cache_size = (size_t)c.max_cache_size;
    o.enable_mixed_precision = c.enable_mixed_precision != 0;
    o.memory_optimization_level = (uint8_t)c.memory_optimization_level;
    o.enable_simd = c.enable_simd != 0;
    o.activation = c.activation == 1 ? ActivationMode::Int8 : ActivationMode::Ternary;
    o.strict_reference_sum = c.strict_reference_sum != 0;
    o.device = c.device;
    return o;
}

void to_c(const BitNetProviderConfig &c, rbp_config *o) {
    o->quantization_method = c.quantization_method.kind == QuantizationMethod::Binary    ? 0
                             : c.quantization_method.kind == QuantizationMethod::Ternary ? 1
                                                                                         : 2;
    o->enable_kernel_caching = c.enable_kernel_caching;
    o->max_cache_size = c.max_cache_size;
    o->enable_mixed_precision = c.enable_mixed_precision;
    o->memory_optimization_level = c.memory_optimization_level;
    o->enable_simd = c.enable_simd;
    o->activation = c.activation == ActivationMode::Int8 ? 1 : 0;
    o->strict_reference_sum = c.strict_reference_sum;
    o->device = c.device;
}

Tensor make_tensor(const float *data, const uint64_t *shape, int ndim, int dtype) {
    std::vector<size_t> sh(shape, shape + ndim);
    size_t count = 1;
    for (size_t d : sh) count *= d;
    return Tensor::from_data(std::vector<float>(data, data + count), sh, (DataType)dtype,
                             TensorLayout::RowMajor);
}
}  // namespace

extern "C" {

const char *rbp_last_error(void) { return g_err.c_str(); }

void rbp_default_config(rbp_config *cfg) {
    if (cfg) to_c(BitNetProviderConfig{}, cfg);
}

int rbp_provider_create(const rbp_config *cfg, rbp_provider **out) {
    return guarded([&] {
        if (!out) throw Error("out is NULL");
        *out = nullptr;
        BitNetProviderConfig c = cfg ? to_cpp(*cfg) : BitNetProviderConfig{};
        rbp_provider *h = new rbp_provider();
        try {
            h->p = std::make_shared<BitNetExecutionProvider>(c);
            h->quantizer.reset(new BitNetQuantizer(
                c.quantization_method, h->p->device(),
                c.strict_reference_sum ? RBN_SUM_STRICT_SEQ : RBN_SUM_TREE));
        } catch (...) {
            delete h;
            throw;
        }
        *out = h;
    });
}

int rbp_provider_destroy(rbp_provider *p) {
    delete p;
    return RBP_OK;
}

int rbp_provider_id(rbp_provider *p) { return p ? (int)p->p->provider_id().kind : -1; }

int rbp_provider_get_config(rbp_provider *p, rbp_config *out) {
    return guarded([&] {
        if (!p || !out) throw Error("null argument");
        to_c(p->p->get_config(), out);
    });
}

int rbp_provider_supports(rbp_provider *p, const char *op_type) {
    if (!p || !op_type) return 0;
    OperatorSpec spec;
    spec.op_type = op_type;
    return p->p->can_handle({spec})[0] ? 1 : 0;
}

float rbp_provider_estimate_speedup(rbp_provider *p, const char *op_type) {
    if (!p || !op_type) return 0.0f;
    OperatorSpec spec;
    spec.op_type = op_type;
    return p->p->estimate_speedup(spec);
}

int rbp_provider_capability(rbp_provider *p, int *n_ops, int *performance_profile) {
    return guarded([&] {
        if (!p) throw Error("provider is NULL");
        ProviderCapability c = p->p->get_capability();
        if (n_ops) *n_ops = (int)c.supported_ops.size();
        if (performance_profile) *performance_profile = (int)c.performance_profile;
    });
}

int rbp_provider_has_data_type(rbp_provider *p, int dtype) {
    if (!p) return 0;
    for (DataType d : p->p->get_capability().data_types)
        if ((int)d == dtype) return 1;
    return 0;
}

int rbp_provider_configure(rbp_provider *p, uint64_t memory_limit, int optimization_level,
                           const char *const *keys, const char *const *values, int n) {
    return guarded([&] {
        if (!p) throw Error("provider is NULL");
        ProviderConfig c;
        c.has_memory_limit = memory_limit != 0;
        c.memory_limit = (size_t)memory_limit;
        c.optimization_level = (OptimizationLevel)optimization_level;
        for (int i = 0; i < n; ++i) c.custom_options[keys[i]] = values[i];
        p->p->configure(c);
    });
}

int rbp_provider_shutdown(rbp_provider *p) {
    return guarded([&] {
        if (!p) throw Error("provider is NULL");
        p->p->shutdown();
    });
}

int rbp_provider_compile_subgraph(rbp_provider *p, const char *const *op_types, int n_nodes,
                                  rbp_kernel **out) {
    return guarded([&] {
        if (!p || !out) throw Error("null argument");
        *out = nullptr;
        SubGraph g;
        for (int i = 0; i < n_nodes; ++i) {
            GraphNode node;
            node.id = (size_t)i;
            node.op_type = op_types[i];
            node.inputs = {"A", "B"};
            node.outputs = {"C"};
            g.nodes.push_back(node);
        }
        g.inputs = {"A", "B"};
        g.outputs = {"C"};
        rbp_kernel *k = new rbp_kernel();
        try {
            k->k = p->p->compile_subgraph(g);
        } catch (...) {
            delete k;
            throw;
        }
        *out = k;
    });
}

int rbp_allocate(rbp_provider *p, const uint64_t *shape, int ndim, int dtype, void **d_ptr,
                 uint64_t *size, uint64_t *alignment) {
    return guarded([&] {
        if (!p || !d_ptr) throw Error("null argument");
        std::vector<size_t> sh(shape, shape + ndim);
        TensorBuffer b = p->p->get_allocator()->allocate(sh, (DataType)dtype);
        *d_ptr = b.ptr;
        if (size) *size = b.size;
        if (alignment) *alignment = b.alignment;
    });
}

int rbp_deallocate(rbp_provider *p, void *d_ptr, uint64_t size, uint64_t alignment) {
    return guarded([&] {
        if (!p) throw Error("provider is NULL");
        TensorBuffer b;
        b.ptr = (uint8_t *)d_ptr;
        b.size = (size_t)size;
        b.alignment = (size_t)alignment;
        b.memory_type = MemoryType::DeviceMemory;
        p->p->get_allocator()->deallocate(b);
    });
}

int rbp_provider_memory_stats(rbp_provider *p, uint64_t *binary_tensor_count,
                              uint64_t *ternary_tensor_count, uint64_t *memory_saved_bytes,
                              float *average_compression_ratio) {
    return guarded([&] {
        if (!p) throw Error("provider is NULL");
        const BitNetMemoryStats &s = p->p->get_memory_stats();
        if (binary_tensor_count) *binary_tensor_count = s.binary_tensor_count;
        if (ternary_tensor_count) *ternary_tensor_count = s.ternary_tensor_count;
        if (memory_saved_bytes) *memory_saved_bytes = s.memory_saved_bytes;
        if (average_compression_ratio) *average_compression_ratio = s.average_compression_ratio;
    });
}

int rbp_memory_info(rbp_provider *p, uint64_t *total, uint64_t *allocated, uint64_t *peak) {
    return guarded([&] {
        if (!p) throw Error("provider is NULL");
        MemoryInfo i = p->p->get_allocator()->get_memory_info();
        if (total) *total = i.total_bytes;
        if (allocated) *allocated = i.allocated_bytes;
        if (peak) *peak = i.peak_bytes;
    });
}

int rbp_create_ternary_matmul_kernel(rbp_provider *p, uint64_t m, uint64_t n, uint64_t k,
                                     rbp_kernel **out) {
    return guarded([&] {
        if (!p || !out) throw Error("null argument");
        rbp_kernel *h = new rbp_kernel();
        h->k = create_ternary_matmul_kernel((size_t)m, (size_t)n, (size_t)k, p->p->device());
        *out = h;
    });
}

int rbp_kernel_destroy(rbp_kernel *k) {
    delete k;
    return RBP_OK;
}

int rbp_kernel_execute(rbp_kernel *k, int n_inputs, const float *const *h_data,
                       const uint64_t *const *shapes, const int *ndims, const int *dtypes,
                       float *h_out, uint64_t out_capacity, uint64_t out_shape[2]) {
    return guarded([&] {
        if (!k) throw Error("kernel is NULL");
        std::vector<Tensor> inputs;
        for (int i = 0; i < n_inputs; ++i)
            inputs.push_back(make_tensor(h_data[i], shapes[i], ndims[i], dtypes[i]));
        std::vector<Tensor> results = k->k->execute(inputs);
        const Tensor &r = results.at(0);
        if (r.numel() > out_capacity) throw Error("output buffer too small");
        std::copy(r.to_vec().begin(), r.to_vec().end(), h_out);
        if (out_shape) {
            out_shape[0] = r.shape().size() > 0 ? r.shape()[0] : 0;
            out_shape[1] = r.shape().size() > 1 ? r.shape()[1] : 0;
        }
    });
}

int rbp_kernel_execute_group(rbp_kernel *k, int n_pairs, const float *const *h_a,
                             const float *const *h_b, const uint64_t shape_a[2],
                             const uint64_t shape_b[2], float *const *h_out,
                             uint64_t out_capacity_each, int *launches) {
    return guarded([&] {
        if (!k || !h_a || !h_b || !shape_a || !shape_b || !h_out) throw Error("null argument");
        if (n_pairs < 1) throw Error("Ternary MatMul group requires pairs of inputs (A_i, B_i)");
        auto *bk = dynamic_cast<BitNetKernel *>(k->k.get());
        if (!bk) throw Error("not a BitNet kernel");
        std::vector<Tensor> inputs;
        for (int i = 0; i < n_pairs; ++i) {
            inputs.push_back(make_tensor(h_a[i], shape_a, 2, 0));
            inputs.push_back(make_tensor(h_b[i], shape_b, 2, 0));
        }
        std::vector<Tensor> results = bk->execute_group(inputs, launches);
        for (int i = 0; i < n_pairs; ++i) {
            const Tensor &r = results.at((size_t)i);
            if (r.numel() > out_capacity_each) throw Error("output buffer too small");
            if (!h_out[i]) throw Error("null argument");
            std::copy(r.to_vec().begin(), r.to_vec().end(), h_out[i]);
        }
    });
}

int rbp_kernel_stats(rbp_kernel *k, uint64_t *execution_count, double *average_us, double *min_us,
                     double *max_us) {
    return guarded([&] {
        if (!k) throw Error("kernel is NULL");
        KernelStats s = k->k->get_performance_stats();
        if (execution_count) *execution_count = s.execution_count;
        if (average_us) *average_us = s.average_time_us;
        if (min_us) *min_us = s.min_time_us;
        if (max_us) *max_us = s.max_time_us;
    });
}

int rbp_kernel_memory_usage(rbp_kernel *k, uint64_t *peak, uint64_t *current,
                            uint64_t *allocations) {
    return guarded([&] {
        if (!k) throw Error("kernel is NULL");
        MemoryUsage u = k->k->get_memory_usage();
        if (peak) *peak = u.peak_bytes;
        if (current) *current = u.current_bytes;
        if (allocations) *allocations = u.allocation_count;
    });
}

int rbp_quantize_ternary(rbp_provider *p, const float *h_data, const uint64_t *shape, int ndim,
                         int dtype, rbp_ternary **out) {
    return guarded([&] {
        if (!p || !out) throw Error("null argument");
        *out = nullptr;
        Tensor t = make_tensor(h_data, shape, ndim, dtype);
        rbp_ternary *h = new rbp_ternary();
        try {
            h->t = p->quantizer->quantize_ternary(t);
        } catch (...) {
            delete h;
            throw;
        }
        *out = h;
    });
}

int rbp_ternary_destroy(rbp_ternary *t) {
    delete t;
    return RBP_OK;
}

int rbp_ternary_info(rbp_ternary *t, float *scale, float *threshold, uint64_t *element_count,
                     uint64_t *memory_size, float *compression_ratio) {
    return guarded([&] {
        if (!t) throw Error("tensor is NULL");
        if (scale) *scale = t->t.scale;
        if (threshold) *threshold = t->t.threshold;
        if (element_count) *element_count = t->t.element_count;
        if (memory_size) *memory_size = t->t.memory_size();
        if (compression_ratio) *compression_ratio = t->t.memory_size() ? t->t.compression_ratio() : 0.0f;
    });
}

int rbp_ternary_packed(rbp_ternary *t, uint8_t *h_out, uint64_t capacity) {
    return guarded([&] {
        if (!t || !h_out) throw Error("null argument");
        if (capacity < t->t.packed_data.size()) throw Error("buffer too small");
        std::copy(t->t.packed_data.begin(), t->t.packed_data.end(), h_out);
    });
}

int rbp_ternary_from_parts(const uint8_t *h_packed, uint64_t packed_bytes, const uint64_t *shape,
                           int ndim, float scale, float threshold, rbp_ternary **out) {
    return guarded([&] {
        if (!out || (!h_packed && packed_bytes) || (!shape && ndim > 0)) throw Error("null argument");
        if (ndim < 0 || ndim > 8) throw Error("ndim must be in [0, 8]");
        auto t = std::make_unique<rbp_ternary>();
        t->t.packed_data.assign(h_packed, h_packed + packed_bytes);
        size_t n = 1;
        for (int i = 0; i < ndim; ++i) {
            t->t.shape.push_back((size_t)shape[i]);
            n *= (size_t)shape[i];
        }
        t->t.element_count = n;
        t->t.scale = scale;
        t->t.threshold = threshold;
        validate_ternary_tensor(t->t);
        *out = t.release();
    });
}

int rbp_ternary_shape(rbp_ternary *t, uint64_t shape[8], int *ndim) {
    return guarded([&] {
        if (!t || !shape || !ndim) throw Error("null argument");
        *ndim = (int)t->t.shape.size();
        for (size_t i = 0; i < t->t.shape.size() && i < 8; ++i) shape[i] = t->t.shape[i];
    });
}

int rbp_ternary_save(rbp_ternary *t, const char *path) {
    return guarded([&] {
        if (!t || !path) throw Error("null argument");
        save_ternary_tensor(t->t, path);
    });
}

int rbp_ternary_load(const char *path, rbp_ternary **out) {
    return guarded([&] {
        if (!path || !out) throw Error("null argument");
        auto t = std::make_unique<rbp_ternary>();
        t->t = load_ternary_tensor(path);
        *out = t.release();
    });
}

int rbp_kernel_execute_prepacked(rbp_kernel *k, const float *h_a, const uint64_t *shape_a, int ndim_a,
                                 rbp_ternary *w, float *h_out, uint64_t out_capacity,
                                 uint64_t out_shape[2]) {
    return guarded([&] {
        if (!k || !w || !h_out) throw Error("null argument");
        auto *bk = dynamic_cast<BitNetKernel *>(k->k.get());
        if (!bk) throw Error("not a BitNet kernel");
        Tensor r = bk->execute_prepacked(make_tensor(h_a, shape_a, ndim_a, 0), w->t);
        if (r.numel() > out_capacity) throw Error("output buffer too small");
        std::copy(r.to_vec().begin(), r.to_vec().end(), h_out);
        if (out_shape) {
            out_shape[0] = r.shape()[0];
            out_shape[1] = r.shape()[1];
        }
    });
}

int rbp_ternary_get_value(rbp_ternary *t, uint64_t index) {
    return t ? (int)t->t.get_value((size_t)index) : 0;
}

int rbp_dequantize_ternary(rbp_provider *p, rbp_ternary *t, float *h_out, uint64_t capacity) {
    return guarded([&] {
        if (!p || !t || !h_out) throw Error("null argument");
        Tensor r = p->quantizer->dequantize_ternary(t->t);
        if (r.numel() > capacity) throw Error("buffer too small");
        std::copy(r.to_vec().begin(), r.to_vec().end(), h_out);
    });
}

}  // extern "C"
