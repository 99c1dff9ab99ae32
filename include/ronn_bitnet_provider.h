/*
 * ronn_bitnet_provider.h - C ABI over the host-side provider mirror
 * (ronn_amd/csrc/host/bitnet_provider.hpp), for bindings that want the reference's
 * provider-level objects rather than the kernel-level calls of ronn_bitnet_hip.h.
 * Exported by the same shared library.
 *
 * Every function returns 0 or a negative status; rbp_last_error() has the message of
 * the calling thread's last failure, which for provider-level errors is the same text
 * the reference's anyhow::Error carries (citations below are relative to
 * crates/ronn-providers/src/bitnet/).
 */
#ifndef RONN_BITNET_PROVIDER_H
#define RONN_BITNET_PROVIDER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rbp_provider rbp_provider;
typedef struct rbp_kernel rbp_kernel;
typedef struct rbp_ternary rbp_ternary;

#define RBP_OK 0
#define RBP_ERR -1 /* a ronn::Error was raised; see rbp_last_error() */

/* BitNetProviderConfig (provider.rs:41-55) plus this build's two additions. */
typedef struct rbp_config {
    int quantization_method; /* 0 = Binary, 1 = Ternary, 2 = AsymmetricBinary */
    int enable_kernel_caching;
    uint64_t max_cache_size;
    int enable_mixed_precision;
    int memory_optimization_level;
    int enable_simd;
    int activation;           /* 0 = ternary (reference), 1 = int8 per token */
    int strict_reference_sum; /* 1 = bit-exact sequential f32 sums, 0 = f64 tree */
    int device;
} rbp_config;

const char *rbp_last_error(void);

/* create_bitnet_provider / create_bitnet_provider_with_config (provider.rs:389-398).
 * cfg == NULL gives the defaults. */
void rbp_default_config(rbp_config *cfg);
int rbp_provider_create(const rbp_config *cfg, rbp_provider **out);
int rbp_provider_destroy(rbp_provider *p);
/* ProviderId as the declaration index of types.rs:24-35 (BitNet = 3). */
int rbp_provider_id(rbp_provider *p);
int rbp_provider_get_config(rbp_provider *p, rbp_config *out);
/* supports_operation / can_handle (provider.rs:127-129, :273-278): 1 or 0. */
int rbp_provider_supports(rbp_provider *p, const char *op_type);
float rbp_provider_estimate_speedup(rbp_provider *p, const char *op_type);
/* get_capability (provider.rs:250-271): number of supported ops, the performance profile
 * (2 = MemoryOptimized) and whether a DataType code is listed. */
int rbp_provider_capability(rbp_provider *p, int *n_ops, int *performance_profile);
int rbp_provider_has_data_type(rbp_provider *p, int dtype);
/* configure (provider.rs:316-364).  memory_limit 0 = None; optimization_level
 * 0 None, 1 Basic, 2 Aggressive, 3 Custom; n key/value pairs of custom_options. */
int rbp_provider_configure(rbp_provider *p, uint64_t memory_limit, int optimization_level,
                           const char *const *keys, const char *const *values, int n);
int rbp_provider_shutdown(rbp_provider *p);
/* compile_subgraph (provider.rs:280-310) for a subgraph of n_nodes nodes with these op types. */
int rbp_provider_compile_subgraph(rbp_provider *p, const char *const *op_types, int n_nodes,
                                  rbp_kernel **out);
/* get_allocator + TensorAllocator (allocator.rs:99-149): device memory. */
int rbp_allocate(rbp_provider *p, const uint64_t *shape, int ndim, int dtype, void **d_ptr,
                 uint64_t *size, uint64_t *alignment);
int rbp_deallocate(rbp_provider *p, void *d_ptr, uint64_t size, uint64_t alignment);
int rbp_memory_info(rbp_provider *p, uint64_t *total, uint64_t *allocated, uint64_t *peak);
/* get_memory_stats (provider.rs:121-123) -> BitNetMemoryStats (allocator.rs:157-205); any
 * out-pointer may be NULL. */
int rbp_provider_memory_stats(rbp_provider *p, uint64_t *binary_tensor_count,
                              uint64_t *ternary_tensor_count, uint64_t *memory_saved_bytes,
                              float *average_compression_ratio);

/* create_ternary_matmul_kernel(m, n, k) (kernels.rs:339-344) on the provider's device. */
int rbp_create_ternary_matmul_kernel(rbp_provider *p, uint64_t m, uint64_t n, uint64_t k,
                                     rbp_kernel **out);
int rbp_kernel_destroy(rbp_kernel *k);
/* CompiledKernel::execute (kernels.rs:255-319).  n_inputs tensors, each a host f32
 * buffer with its shape and DataType code.  The single result is written to h_out
 * (capacity in elements); out_shape receives [m, n]. */
int rbp_kernel_execute(rbp_kernel *k, int n_inputs, const float *const *h_data,
                       const uint64_t *const *shapes, const int *ndims, const int *dtypes,
                       float *h_out, uint64_t out_capacity, uint64_t out_shape[2]);
/* Several independent TernaryMatMul nodes of one shape in one call: n_pairs pairs
 * (A_i [m,k], B_i [k,n]), host f32 buffers; h_out[i] (capacity out_capacity_each elements)
 * receives what rbp_kernel_execute gives for {A_i, B_i}, bit for bit.  The reference runs such
 * nodes one execute() at a time (kernels.rs:254-319, issued per node by
 * ProviderRegistry::compile_subgraph, registry.rs:237-266); here the nodes a graph holds side
 * by side (q/k/v or gate/up projections of one token, one layer of several sequences) share
 * one launch in the decode regime (rbn_gemv_t2_i8_grouped, up to RBN_GEMV_GROUP_MAX per
 * launch); nodes that pass the same A are quantised once.  *launches (optional) receives the
 * number of matmul launches issued.  Errors as rbp_kernel_execute, plus a message naming the
 * node whose shape differs from node 0's. */
int rbp_kernel_execute_group(rbp_kernel *k, int n_pairs, const float *const *h_a,
                             const float *const *h_b, const uint64_t shape_a[2],
                             const uint64_t shape_b[2], float *const *h_out,
                             uint64_t out_capacity_each, int *launches);
/* get_performance_stats / get_memory_usage (kernels.rs:321-327). */
int rbp_kernel_stats(rbp_kernel *k, uint64_t *execution_count, double *average_us, double *min_us,
                     double *max_us);
int rbp_kernel_memory_usage(rbp_kernel *k, uint64_t *peak, uint64_t *current, uint64_t *allocations);

/* BitNetQuantizer::quantize_ternary / dequantize_ternary and TernaryTensor
 * (quantization.rs:67-109, :182-207, :249-292). */
int rbp_quantize_ternary(rbp_provider *p, const float *h_data, const uint64_t *shape, int ndim,
                         int dtype, rbp_ternary **out);
int rbp_ternary_destroy(rbp_ternary *t);
int rbp_ternary_info(rbp_ternary *t, float *scale, float *threshold, uint64_t *element_count,
                     uint64_t *memory_size, float *compression_ratio);
int rbp_ternary_packed(rbp_ternary *t, uint8_t *h_out, uint64_t capacity);
int rbp_ternary_get_value(rbp_ternary *t, uint64_t index);
int rbp_dequantize_ternary(rbp_provider *p, rbp_ternary *t, float *h_out, uint64_t capacity);

/* Packed-weight files: ternarisation as a one-time offline step.  The reference has
 * TernaryTensor's fields (quantization.rs:249-260) and no serialisation; the format is
 * this build's ("RBNTERN1", version, shape, scale, threshold, packed bytes in the
 * reference's layout, CRC-32; see csrc/host/bitnet_provider.hpp).  None of these
 * needs a GPU. */
int rbp_ternary_from_parts(const uint8_t *h_packed, uint64_t packed_bytes, const uint64_t *shape,
                           int ndim, float scale, float threshold, rbp_ternary **out);
int rbp_ternary_shape(rbp_ternary *t, uint64_t shape[8], int *ndim);
int rbp_ternary_save(rbp_ternary *t, const char *path);
int rbp_ternary_load(const char *path, rbp_ternary **out);
/* TernaryMatMul with weights that are already ternarised: A [m,k] f32 (host) is
 * quantised as rbp_kernel_execute does, B [k,n] comes from `w`. */
int rbp_kernel_execute_prepacked(rbp_kernel *k, const float *h_a, const uint64_t *shape_a, int ndim_a,
                                 rbp_ternary *w, float *h_out, uint64_t out_capacity,
                                 uint64_t out_shape[2]);

#ifdef __cplusplus
}
#endif
#endif /* RONN_BITNET_PROVIDER_H */
