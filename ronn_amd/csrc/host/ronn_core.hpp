// Host-side mirror of the part of the reference's ronn-core that the BitNet provider
// touches (crates/ronn-core/src/types.rs and tensor.rs): identifiers, data types, the
// host tensor, graph fragments and the three interfaces a provider implements.
// Names, argument meaning and error texts follow the reference so that code and
// tests written against it read the same here.  anyhow::Error becomes ronn::Error.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

namespace ronn {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// types.rs:24-35
struct ProviderId {
    enum Kind { CPU = 0, GPU = 1, WebAssembly = 2, BitNet = 3, Custom = 4 };
    Kind kind = CPU;
    uint32_t custom = 0;
    bool operator==(const ProviderId &o) const { return kind == o.kind && custom == o.custom; }
};
using ProviderType = ProviderId;  // types.rs:20

// types.rs:39-60 (declaration order is the numeric code used across the C ABI)
enum class DataType { F32 = 0, F16, BF16, I8, I32, I64, U8, U32, Bool, F64 };

enum class TensorLayout { RowMajor, ColumnMajor };  // types.rs:77-82

// tensor.rs:40-83, :165, :170, :217-267: the four operations the provider uses.
class Tensor {
   public:
    static Tensor from_data(std::vector<float> data, std::vector<size_t> shape, DataType dtype,
                            TensorLayout layout) {
        size_t count = 1;
        for (size_t d : shape) count *= d;
        if (count != data.size())
            throw Error("shape mismatch: " + std::to_string(data.size()) +
                        " values for a tensor of " + std::to_string(count) + " elements");
        Tensor t;
        t.data_ = std::move(data);
        t.shape_ = std::move(shape);
        t.dtype_ = dtype;
        t.layout_ = layout;
        return t;
    }
    const std::vector<size_t> &shape() const { return shape_; }
    DataType dtype() const { return dtype_; }
    TensorLayout layout() const { return layout_; }
    size_t numel() const { return data_.size(); }
    // Row-major flattening, as Candle's flatten_all gives (tensor.rs:219-229).
    const std::vector<float> &to_vec() const { return data_; }

   private:
    std::vector<float> data_;
    std::vector<size_t> shape_;
    DataType dtype_ = DataType::F32;
    TensorLayout layout_ = TensorLayout::RowMajor;
};

// types.rs:121-135, :139-150, :348-358, :335-345
struct GraphNode {
    size_t id = 0;
    std::string op_type;
    std::map<std::string, std::string> attributes;
    std::vector<std::string> inputs, outputs;
    std::string name;
};
struct GraphEdge {
    size_t from_node = 0, to_node = 0;
    std::string tensor_name;
    std::vector<size_t> tensor_shape;
    DataType tensor_dtype = DataType::F32;
};
struct SubGraph {
    std::vector<GraphNode> nodes;
    std::vector<GraphEdge> edges;
    std::vector<std::string> inputs, outputs;
};
struct OperatorSpec {
    std::string op_type;
    std::vector<DataType> input_types, output_types;
    std::map<std::string, std::string> attributes;
};

// types.rs:168-189
struct MemoryUsage {
    size_t peak_bytes = 0, current_bytes = 0, allocation_count = 0;
};
struct KernelStats {
    uint64_t execution_count = 0;
    double average_time_us = 0.0, min_time_us = 0.0, max_time_us = 0.0;
};

// types.rs:231-265
enum class MemoryType { SystemRAM, DeviceMemory, SharedMemory, MappedMemory };
enum class PerformanceProfile { CPU, GPU, MemoryOptimized, PowerEfficient };
struct ResourceRequirements {
    bool has_min_memory = false;
    size_t min_memory_bytes = 0;
    std::vector<std::string> cpu_features;
    bool has_gpu_memory = false;
    size_t gpu_memory_bytes = 0;
};
struct ProviderCapability {
    std::set<std::string> supported_ops;
    std::vector<DataType> data_types;
    std::vector<MemoryType> memory_types;
    PerformanceProfile performance_profile = PerformanceProfile::CPU;
    ResourceRequirements resource_requirements;
};

// types.rs:268-291
enum class OptimizationLevel { None, Basic, Aggressive, Custom };
struct ProviderConfig {
    bool has_thread_count = false;
    size_t thread_count = 0;
    bool has_memory_limit = false;
    size_t memory_limit = 0;
    OptimizationLevel optimization_level = OptimizationLevel::Basic;
    std::map<std::string, std::string> custom_options;
};

// types.rs:306-332
struct TensorBuffer {
    uint8_t *ptr = nullptr;
    size_t size = 0, alignment = 0;
    MemoryType memory_type = MemoryType::SystemRAM;
};
struct MemoryInfo {
    size_t total_bytes = 0, allocated_bytes = 0, peak_bytes = 0;
};

// types.rs:153-165.  Send + Sync in the reference: execute() may be called from many
// threads, so implementations guard their interior state.
class CompiledKernel {
   public:
    virtual ~CompiledKernel() = default;
    virtual std::vector<Tensor> execute(const std::vector<Tensor> &inputs) = 0;
    virtual MemoryUsage get_memory_usage() const = 0;
    virtual KernelStats get_performance_stats() const = 0;
};

// types.rs:294-303
class TensorAllocator {
   public:
    virtual ~TensorAllocator() = default;
    virtual TensorBuffer allocate(const std::vector<size_t> &shape, DataType dtype) = 0;
    virtual void deallocate(const TensorBuffer &buffer) = 0;
    virtual MemoryInfo get_memory_info() const = 0;
};

// types.rs:192-213
class ExecutionProvider {
   public:
    virtual ~ExecutionProvider() = default;
    virtual ProviderId provider_id() const = 0;
    virtual ProviderCapability get_capability() const = 0;
    virtual std::vector<bool> can_handle(const std::vector<OperatorSpec> &operators) const = 0;
    virtual std::unique_ptr<CompiledKernel> compile_subgraph(const SubGraph &subgraph) = 0;
    virtual std::shared_ptr<TensorAllocator> get_allocator() const = 0;
    virtual void configure(const ProviderConfig &config) = 0;
    virtual void shutdown() = 0;
};

}  // namespace ronn
