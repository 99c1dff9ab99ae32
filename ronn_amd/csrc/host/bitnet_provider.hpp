// MI355X BitNet execution provider: the host side of the drop-in, written against the
// C ABI in include/ronn_bitnet_hip.h.  It mirrors the reference's
// crates/ronn-providers/src/bitnet/{quantization,kernels,provider,allocator}.rs:
// same type and function names, same argument meaning, same error texts, so the
// parity tests read like the reference's own.  Only the ternary path is implemented;
// the binary (XNOR) half of the reference raises an error that says so.
//
// Deliberate differences from the reference, all on the host side:
//   - TernaryMatMul kernels take m, n, k from the inputs at execute() time unless
//     they were created with explicit dimensions (the reference hard-codes 64x64x64
//     in provider.rs:157-159 and rejects everything else).
//   - The weight operand (input 1) is ternarised once and cached by content hash; the
//     reference re-ternarises it on every call (kernels.rs:278).
//   - KernelStats are really updated (the reference measures and drops them,
//     kernels.rs:313-316).
//   - The default quantisation method is Ternary (the reference defaults to Binary,
//     provider.rs:60).
#pragma once

#include <atomic>
#include <mutex>
#include <set>
#include <unordered_map>

#include "../../../include/ronn_bitnet_hip.h"
#include "ronn_core.hpp"

namespace ronn {
namespace bitnet {

// quantization.rs:13-20
struct QuantizationMethod {
    enum Kind { Binary, Ternary, AsymmetricBinary } kind = Ternary;
    float threshold = 0.0f;  // AsymmetricBinary only
    bool operator==(const QuantizationMethod &o) const { return kind == o.kind; }
};

// How activations (input 0) are quantised.
enum class ActivationMode {
    Ternary,  // as the reference: quantize_ternary over the whole tensor (kernels.rs:277)
    Int8      // per-token absmax int8 (no reference counterpart; faster, finer)
};

// One device context shared by everything a provider creates.
class Device {
   public:
    explicit Device(int index);
    ~Device();
    Device(const Device &) = delete;
    Device &operator=(const Device &) = delete;
    rbn_ctx *ctx() const { return ctx_; }
    int index() const { return index_; }

   private:
    rbn_ctx *ctx_ = nullptr;
    int index_ = 0;
};

// Throws ronn::Error carrying rbn_last_error() when rc != RBN_OK.
void check(int rc, const char *what);

// quantization.rs:249-292
struct TernaryTensor {
    std::vector<uint8_t> packed_data;
    std::vector<size_t> shape;
    float scale = 1.0f;
    float threshold = 0.0f;
    size_t element_count = 0;

    size_t memory_size() const { return packed_data.size(); }
    float compression_ratio() const {
        return (float)(element_count * sizeof(float)) / (float)memory_size();
    }
    int8_t get_value(size_t index) const;
};

// Packed-weight file: ternarisation becomes a one-time offline step.  The reference has the
// fields (quantization.rs:249-260) but no serialisation; the format is this build's:
//   0  "RBNTERN1"            8 bytes
//   8  u32 version (1)      12  u32 ndim (<= 8)
//  16  u64 element_count    24  f32 scale     28  f32 threshold
//  32  u64 packed_bytes (= ceil(element_count / 4))
//  40  u64 shape[ndim]      then the packed bytes (reference layout), then
//  u32 CRC-32 (IEEE) of everything before it.  Little-endian throughout.
void save_ternary_tensor(const TernaryTensor &t, const std::string &path);
TernaryTensor load_ternary_tensor(const std::string &path);
// Checks the invariants that quantize_ternary guarantees (sizes, zero tail bits).
void validate_ternary_tensor(const TernaryTensor &t);

// quantization.rs:24-208 (ternary half)
class BitNetQuantizer {
   public:
    BitNetQuantizer(QuantizationMethod method, std::shared_ptr<Device> device,
                    int sum_mode = RBN_SUM_STRICT_SEQ)
        : method_(method), device_(std::move(device)), sum_mode_(sum_mode) {}
    TernaryTensor quantize_ternary(const Tensor &input) const;
    Tensor dequantize_ternary(const TernaryTensor &t) const;
    QuantizationMethod method() const { return method_; }

   private:
    QuantizationMethod method_;
    std::shared_ptr<Device> device_;
    int sum_mode_;
};

// kernels.rs:17-32
struct BitNetOperation {
    enum Kind { BinaryMatMul, TernaryMatMul, BinaryElementWise, QuantizedBatchNorm } kind;
    size_t m = 0, n = 0, k = 0;  // 0,0,0 = take the dimensions from the inputs
};

// kernels.rs:36-47, :254-328
class BitNetKernel : public CompiledKernel {
   public:
    BitNetKernel(BitNetOperation operation, QuantizationMethod method,
                 std::shared_ptr<Device> device, ActivationMode act_mode, int sum_mode,
                 bool cache_weights, size_t max_cache_bytes);
    ~BitNetKernel() override;
    std::vector<Tensor> execute(const std::vector<Tensor> &inputs) override;
    // TernaryMatMul with weights that are already ternarised (e.g. loaded from a packed
    // weight file): A [m,k] f32 is quantised as in execute(), B comes from `w` ([k,n]).
    Tensor execute_prepacked(const Tensor &a, const TernaryTensor &w);
    // Several independent TernaryMatMul nodes of ONE shape in one call: inputs are the pairs
    // (A_0, B_0, A_1, B_1, ...), every A_i [m,k] and every B_i [k,n]; result i is what
    // execute({A_i, B_i}) returns, bit for bit.  These are the nodes a graph holds side by side
    // (the q/k/v or gate/up projections of one token, the same layer of several sequences) and
    // that ProviderRegistry::compile_subgraph (registry.rs:237-266) would otherwise run one by
    // one.  In the decode regime (the shapes rbn_matmul_t2_i8 gives to the GEMV) up to
    // RBN_GEMV_GROUP_MAX of them become ONE launch of rbn_gemv_t2_i8_grouped, which shares the
    // fixed cost of a launch between them; other shapes run one launch per node.
    // *launches (optional) receives the number of matmul launches issued.
    std::vector<Tensor> execute_group(const std::vector<Tensor> &inputs, int *launches = nullptr);
    MemoryUsage get_memory_usage() const override;
    KernelStats get_performance_stats() const override;

   private:
    struct CachedWeights {
        void *d_tiled = nullptr;
        float scale = 1.0f;
        size_t bytes = 0;
        // what a hit is confirmed with, besides the 64-bit key: dimensions, byte count of the
        // source and a second, independently computed digest of it
        size_t k = 0, n = 0, source_bytes = 0;
        uint64_t check = 0;
        uint64_t last_use = 0;  // for least-recently-used eviction
    };
    Tensor execute_ternary_matmul(const Tensor &a, const Tensor &b);
    // the shared tail: quantise A, multiply, download
    Tensor multiply(const Tensor &a, size_t m, size_t k, size_t n, const void *d_tiled, float w_scale);
    // tiled device copy of packed weights, cached by `key` when caching is on; *owned tells
    // the caller to free it
    CachedWeights tiled_weights(uint64_t key, uint64_t check, size_t source_bytes, size_t k, size_t n, const uint8_t *h_packed,
                                const float *h_f32, float scale, bool *owned);
    void update_stats(double us);  // kernels.rs:235-251

    BitNetOperation operation_;
    QuantizationMethod method_;
    std::shared_ptr<Device> device_;
    ActivationMode act_mode_;
    int sum_mode_;
    bool cache_weights_;
    size_t max_cache_bytes_;
    mutable std::mutex lock_;
    KernelStats stats_;
    MemoryUsage memory_usage_;
    std::unordered_map<uint64_t, CachedWeights> weight_cache_;
    size_t cache_bytes_ = 0;
    uint64_t use_clock_ = 0;
    // keys of cached matrices a running execute_group still needs: never evicted
    std::set<uint64_t> pinned_;
};

// kernels.rs:339-344.  Explicit dimensions are checked against the inputs exactly as
// the reference does (:142-152).
std::unique_ptr<BitNetKernel> create_ternary_matmul_kernel(size_t m, size_t n, size_t k,
                                                           std::shared_ptr<Device> device);

// allocator.rs:16-149, with device memory behind it.
class BitNetMemoryAllocator : public TensorAllocator {
   public:
    explicit BitNetMemoryAllocator(std::shared_ptr<Device> device);
    TensorBuffer allocate(const std::vector<size_t> &shape, DataType dtype) override;
    void deallocate(const TensorBuffer &buffer) override;
    MemoryInfo get_memory_info() const override;

   private:
    std::shared_ptr<Device> device_;
    std::atomic<size_t> allocated_{0}, peak_{0};
    size_t total_bytes_ = 0;
};

// allocator.rs:157-205
struct BitNetMemoryStats {
    size_t binary_tensor_count = 0, ternary_tensor_count = 0, memory_saved_bytes = 0;
    float average_compression_ratio = 1.0f;
    void add_binary_tensor(size_t original, size_t compressed);
    void add_ternary_tensor(size_t original, size_t compressed);
};

// provider.rs:41-68
struct BitNetProviderConfig {
    QuantizationMethod quantization_method{};  // Ternary here (reference: Binary)
    bool enable_kernel_caching = true;
    size_t max_cache_size = 64u * 1024 * 1024;
    bool enable_mixed_precision = true;
    uint8_t memory_optimization_level = 2;
    bool enable_simd = true;
    // additions of this build, reachable through ProviderConfig.custom_options
    ActivationMode activation = ActivationMode::Ternary;  // "activation" = ternary|int8
    bool strict_reference_sum = true;                     // "strict_reference_sum" = true|false
    int device = 0;
};

// provider.rs:25-38, :70-386
class BitNetExecutionProvider : public ExecutionProvider {
   public:
    BitNetExecutionProvider() : BitNetExecutionProvider(BitNetProviderConfig{}) {}
    explicit BitNetExecutionProvider(const BitNetProviderConfig &config);  // with_config

    const BitNetProviderConfig &get_config() const { return config_; }
    const BitNetMemoryStats &get_memory_stats() const { return memory_stats_; }
    bool supports_operation(const std::string &op_type) const;
    float estimate_speedup(const OperatorSpec &op_spec) const;

    ProviderId provider_id() const override;
    ProviderCapability get_capability() const override;
    std::vector<bool> can_handle(const std::vector<OperatorSpec> &operators) const override;
    std::unique_ptr<CompiledKernel> compile_subgraph(const SubGraph &subgraph) override;
    std::shared_ptr<TensorAllocator> get_allocator() const override;
    void configure(const ProviderConfig &config) override;
    void shutdown() override;

    std::shared_ptr<Device> device() const { return device_; }

   private:
    std::unique_ptr<CompiledKernel> create_kernel_for_operation(const GraphNode &node) const;

    BitNetProviderConfig config_;
    std::shared_ptr<Device> device_;
    std::shared_ptr<TensorAllocator> allocator_;
    std::set<std::string> supported_ops_;
    BitNetMemoryStats memory_stats_;
};

// provider.rs:389-398
std::shared_ptr<ExecutionProvider> create_bitnet_provider();
std::shared_ptr<ExecutionProvider> create_bitnet_provider_with_config(
    const BitNetProviderConfig &config);

}  // namespace bitnet
}  // namespace ronn
