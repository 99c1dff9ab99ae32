//! `ExecutionProvider` with `ProviderId::BitNet` on an MI355X.
//!
//! Stands in for `BitNetExecutionProvider` (crates/ronn-providers/src/bitnet/provider.rs:25-398)
//! and `BitNetMemoryAllocator` (bitnet/allocator.rs:15-149).  The provider object, its
//! configuration rules, its supported-operation set, its speed-up table and its error texts live
//! behind the C ABI (`rbp_provider`), where the GPU tests exercise them; this file converts between
//! the traits' Rust types and that ABI.

use std::collections::HashSet;
use std::ffi::CString;
use std::os::raw::{c_char, c_int, c_void};
use std::ptr::null_mut;
use std::sync::Arc;

use anyhow::{anyhow, Result};
use ronn_bitnet_hip_sys as sys;
use ronn_core::{
    CompiledKernel, DataType, ExecutionProvider, MemoryInfo, MemoryType, OperatorSpec, OptimizationLevel,
    PerformanceProfile, ProviderCapability, ProviderConfig, ProviderId, ResourceRequirements, SubGraph,
    TensorAllocator, TensorBuffer,
};
use tracing::{debug, info};

use crate::hip_kernel::{check, dtype_to_code, null_kernel, HipKernel};

/// provider.rs of the reference takes this from bitnet/quantization.rs:13-20; same variants.
#[derive(Debug, Clone, Copy, PartialEq)]
pub enum QuantizationMethod {
    Binary,
    Ternary,
    AsymmetricBinary { threshold: f32 },
}

/// How input 0 (the activations) is quantised.
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum ActivationMode {
    /// `quantize_ternary` over the whole tensor, as the reference does (kernels.rs:277).
    TernaryPerTensor,
    /// Per-token absmax int8 (no counterpart in the reference).
    Int8PerToken,
}

/// `BitNetProviderConfig` (provider.rs:41-68) plus three fields of this implementation.
#[derive(Debug, Clone)]
pub struct BitNetProviderConfig {
    pub quantization_method: QuantizationMethod,
    pub enable_kernel_caching: bool,
    pub max_cache_size: usize,
    pub enable_mixed_precision: bool,
    pub memory_optimization_level: u8,
    pub enable_simd: bool,
    /// Activation quantisation; the default reproduces the reference.
    pub activation: ActivationMode,
    /// true: thresholds and scales are the reference's sequential f32 sums bit for bit
    /// (quantization.rs:79, :96); false: f64 tree sums (faster, not reference-exact).
    pub strict_reference_sum: bool,
    /// HIP device index.
    pub device: i32,
}

impl BitNetProviderConfig {
    fn to_c(&self) -> sys::rbp_config {
        sys::rbp_config {
            quantization_method: match self.quantization_method {
                QuantizationMethod::Binary => 0,
                QuantizationMethod::Ternary => 1,
                QuantizationMethod::AsymmetricBinary { .. } => 2,
            },
            enable_kernel_caching: self.enable_kernel_caching as c_int,
            max_cache_size: self.max_cache_size as u64,
            enable_mixed_precision: self.enable_mixed_precision as c_int,
            memory_optimization_level: c_int::from(self.memory_optimization_level),
            enable_simd: self.enable_simd as c_int,
            activation: (self.activation == ActivationMode::Int8PerToken) as c_int,
            strict_reference_sum: self.strict_reference_sum as c_int,
            device: self.device as c_int,
        }
    }

    fn from_c(c: &sys::rbp_config) -> Self {
        Self {
            quantization_method: match c.quantization_method {
                0 => QuantizationMethod::Binary,
                2 => QuantizationMethod::AsymmetricBinary { threshold: 0.0 },
                _ => QuantizationMethod::Ternary,
            },
            enable_kernel_caching: c.enable_kernel_caching != 0,
            max_cache_size: c.max_cache_size as usize,
            enable_mixed_precision: c.enable_mixed_precision != 0,
            memory_optimization_level: c.memory_optimization_level as u8,
            enable_simd: c.enable_simd != 0,
            activation: if c.activation != 0 { ActivationMode::Int8PerToken } else { ActivationMode::TernaryPerTensor },
            strict_reference_sum: c.strict_reference_sum != 0,
            device: c.device as i32,
        }
    }
}

impl Default for BitNetProviderConfig {
    /// The library's defaults: as provider.rs:57-68, except that the method is Ternary (the
    /// reference defaults to Binary, :60; only the ternary half exists here).
    fn default() -> Self {
        // SAFETY: plain-old-data out-parameter, filled in full.
        let mut c: sys::rbp_config = unsafe { std::mem::zeroed() };
        unsafe { sys::rbp_default_config(&mut c) };
        Self::from_c(&c)
    }
}

/// `BitNetMemoryStats` (allocator.rs:157-205) as `get_memory_stats` reports it.
#[derive(Debug, Clone, Copy, PartialEq)]
pub struct BitNetMemoryStats {
    pub binary_tensor_count: usize,
    pub ternary_tensor_count: usize,
    pub memory_saved_bytes: usize,
    pub average_compression_ratio: f32,
}

/// Owns the library's provider object.
struct ProviderHandle {
    raw: *mut sys::rbp_provider,
}

// SAFETY: the object's const operations are read-only or go through the device context, which
// takes its own lock for every call; `configure` needs `&mut BitNetExecutionProvider`.
unsafe impl Send for ProviderHandle {}
unsafe impl Sync for ProviderHandle {}

impl Drop for ProviderHandle {
    fn drop(&mut self) {
        // SAFETY: created by rbp_provider_create and not used after this.
        unsafe { sys::rbp_provider_destroy(self.raw) };
    }
}

/// Device-memory `TensorAllocator` with the reference's size and alignment rules
/// (allocator.rs:39-75): U8 = 2-bit ternary, 4 elements per byte; Bool = 1 bit per element.
pub struct BitNetHipAllocator {
    provider: Arc<ProviderHandle>,
}

impl TensorAllocator for BitNetHipAllocator {
    /// allocator.rs:100-128; an unsupported dtype gives the reference's message (:61-64).
    fn allocate(&self, shape: &[usize], dtype: DataType) -> Result<TensorBuffer> {
        let dims: Vec<u64> = shape.iter().map(|&d| d as u64).collect();
        let mut p: *mut c_void = null_mut();
        let (mut size, mut alignment) = (0u64, 0u64);
        // SAFETY: `dims` has `dims.len()` entries; valid out-pointers.
        check(unsafe {
            sys::rbp_allocate(self.provider.raw, dims.as_ptr(), dims.len() as c_int, dtype_to_code(dtype), &mut p,
                              &mut size, &mut alignment)
        })?;
        Ok(TensorBuffer {
            ptr: p.cast(),
            size: size as usize,
            alignment: alignment as usize,
            memory_type: MemoryType::DeviceMemory,
        })
    }

    /// allocator.rs:130-140.
    fn deallocate(&self, buffer: TensorBuffer) -> Result<()> {
        // SAFETY: `buffer` came from `allocate` above.
        check(unsafe {
            sys::rbp_deallocate(self.provider.raw, buffer.ptr.cast(), buffer.size as u64, buffer.alignment as u64)
        })
    }

    /// allocator.rs:142-148.
    fn get_memory_info(&self) -> MemoryInfo {
        let (mut total, mut allocated, mut peak) = (0u64, 0u64, 0u64);
        // SAFETY: valid out-pointers.
        let _ = unsafe { sys::rbp_memory_info(self.provider.raw, &mut total, &mut allocated, &mut peak) };
        MemoryInfo { total_bytes: total as usize, allocated_bytes: allocated as usize, peak_bytes: peak as usize }
    }
}

/// The operation names `get_capability` can report (provider.rs:87-99); which of them the
/// provider supports is the library's answer.
const OP_NAMES: [&str; 12] =
    ["MatMul", "Gemm", "Conv", "Add", "Sub", "Mul", "And", "Or", "Xor", "BatchNormalization", "ReLU", "Sigmoid"];

/// BitNet execution provider backed by the gfx950 kernels.
pub struct BitNetExecutionProvider {
    handle: Arc<ProviderHandle>,
    allocator: Arc<dyn TensorAllocator>,
}

impl BitNetExecutionProvider {
    pub fn new() -> Result<Self> {
        Self::with_config(BitNetProviderConfig::default())
    }

    /// provider.rs:77-114.
    pub fn with_config(config: BitNetProviderConfig) -> Result<Self> {
        info!("Creating BitNet execution provider with method: {:?}", config.quantization_method);
        let c = config.to_c();
        let mut raw = null_mut();
        // SAFETY: valid in- and out-pointers.
        check(unsafe { sys::rbp_provider_create(&c, &mut raw) })?;
        let handle = Arc::new(ProviderHandle { raw });
        let allocator: Arc<dyn TensorAllocator> = Arc::new(BitNetHipAllocator { provider: Arc::clone(&handle) });
        Ok(Self { handle, allocator })
    }

    /// provider.rs:117-119 (by value: the configuration lives in the library).
    pub fn get_config(&self) -> BitNetProviderConfig {
        // SAFETY: plain-old-data out-parameter.
        let mut c: sys::rbp_config = unsafe { std::mem::zeroed() };
        let _ = unsafe { sys::rbp_provider_get_config(self.handle.raw, &mut c) };
        BitNetProviderConfig::from_c(&c)
    }

    /// provider.rs:121-123.
    pub fn get_memory_stats(&self) -> BitNetMemoryStats {
        let (mut binary, mut ternary, mut saved, mut ratio) = (0u64, 0u64, 0u64, 1f32);
        // SAFETY: valid out-pointers.
        let _ = unsafe {
            sys::rbp_provider_memory_stats(self.handle.raw, &mut binary, &mut ternary, &mut saved, &mut ratio)
        };
        BitNetMemoryStats {
            binary_tensor_count: binary as usize,
            ternary_tensor_count: ternary as usize,
            memory_saved_bytes: saved as usize,
            average_compression_ratio: ratio,
        }
    }

    /// provider.rs:127-129.
    pub fn supports_operation(&self, op_type: &str) -> bool {
        match CString::new(op_type) {
            // SAFETY: NUL-terminated string that outlives the call.
            Ok(name) => unsafe { sys::rbp_provider_supports(self.handle.raw, name.as_ptr()) == 1 },
            Err(_) => false,
        }
    }

    /// provider.rs:132-150.
    pub fn estimate_speedup(&self, op_spec: &OperatorSpec) -> f32 {
        match CString::new(op_spec.op_type.as_str()) {
            // SAFETY: as above.
            Ok(name) => unsafe { sys::rbp_provider_estimate_speedup(self.handle.raw, name.as_ptr()) },
            Err(_) => 4.0,
        }
    }

    /// `create_ternary_matmul_kernel(m, n, k)` (kernels.rs:339-344) on this provider's device;
    /// 0, 0, 0 takes the dimensions from the inputs of each call.
    pub fn create_ternary_matmul_kernel(&self, m: usize, n: usize, k: usize) -> Result<HipKernel> {
        let mut raw = null_kernel();
        // SAFETY: valid out-pointer.
        check(unsafe { sys::rbp_create_ternary_matmul_kernel(self.handle.raw, m as u64, n as u64, k as u64, &mut raw) })?;
        Ok(HipKernel::from_raw(raw))
    }
}

impl ExecutionProvider for BitNetExecutionProvider {
    fn provider_id(&self) -> ProviderId {
        ProviderId::BitNet
    }

    /// provider.rs:250-271 with the memory type of this implementation.
    fn get_capability(&self) -> ProviderCapability {
        let supported_ops: HashSet<String> =
            OP_NAMES.iter().filter(|op| self.supports_operation(op)).map(|op| op.to_string()).collect();
        let data_types = [DataType::Bool, DataType::U8, DataType::F32, DataType::F16]
            .into_iter()
            // SAFETY: pure query.
            .filter(|&dt| unsafe { sys::rbp_provider_has_data_type(self.handle.raw, dtype_to_code(dt)) } == 1)
            .collect();
        ProviderCapability {
            supported_ops,
            data_types,
            memory_types: vec![MemoryType::DeviceMemory],
            performance_profile: PerformanceProfile::MemoryOptimized,
            resource_requirements: ResourceRequirements {
                min_memory_bytes: Some(16 * 1024 * 1024),
                cpu_features: vec![],
                gpu_memory_bytes: Some(128 * 1024 * 1024),
            },
        }
    }

    fn can_handle(&self, operators: &[OperatorSpec]) -> Vec<bool> {
        operators.iter().map(|op| self.supports_operation(&op.op_type)).collect()
    }

    /// provider.rs:280-310.  The single-node rule and the messages for unsupported operations
    /// ("BitNet provider currently supports only single-node subgraphs", "Unsupported operation
    /// for BitNet: {op}") are the library's.  The reference's cache lookup can only fail (:289-293,
    /// on a map that is never filled); what is worth caching - the ternarised weights - is cached
    /// inside the kernel object.
    fn compile_subgraph(&self, subgraph: SubGraph) -> Result<Box<dyn CompiledKernel>> {
        debug!("Compiling BitNet subgraph with {} nodes", subgraph.nodes.len());
        let names: Vec<CString> = subgraph
            .nodes
            .iter()
            .map(|node| CString::new(node.op_type.as_str()).map_err(|_| anyhow!("operation name contains NUL")))
            .collect::<Result<_>>()?;
        let ptrs: Vec<*const c_char> = names.iter().map(|n| n.as_ptr()).collect();
        let mut raw = null_kernel();
        // SAFETY: `ptrs` has `ptrs.len()` NUL-terminated strings that outlive the call.
        check(unsafe { sys::rbp_provider_compile_subgraph(self.handle.raw, ptrs.as_ptr(), ptrs.len() as c_int, &mut raw) })?;
        info!("Successfully compiled BitNet kernel for {}", subgraph.nodes[0].op_type);
        Ok(Box::new(HipKernel::from_raw(raw)))
    }

    fn get_allocator(&self) -> Arc<dyn TensorAllocator> {
        Arc::clone(&self.allocator)
    }

    /// provider.rs:316-364.  The library applies `custom_options` at every optimisation level
    /// (the reference parses them only under `Custom`, although its own test sets them under
    /// `Aggressive`, provider.rs:479-500) and knows two more keys: `activation` = ternary | int8
    /// and `strict_reference_sum` = true | false.
    fn configure(&mut self, config: ProviderConfig) -> Result<()> {
        let level = match config.optimization_level {
            OptimizationLevel::None => 0,
            OptimizationLevel::Basic => 1,
            OptimizationLevel::Aggressive => 2,
            OptimizationLevel::Custom => 3,
        };
        let pairs: Vec<(CString, CString)> = config
            .custom_options
            .iter()
            .filter_map(|(k, v)| Some((CString::new(k.as_str()).ok()?, CString::new(v.as_str()).ok()?)))
            .collect();
        let keys: Vec<*const c_char> = pairs.iter().map(|p| p.0.as_ptr()).collect();
        let values: Vec<*const c_char> = pairs.iter().map(|p| p.1.as_ptr()).collect();
        // SAFETY: both arrays have `pairs.len()` NUL-terminated strings that outlive the call.
        check(unsafe {
            sys::rbp_provider_configure(self.handle.raw, config.memory_limit.unwrap_or(0) as u64, level, keys.as_ptr(),
                                        values.as_ptr(), pairs.len() as c_int)
        })?;
        info!("BitNet provider reconfigured with optimization level: {:?}", config.optimization_level);
        Ok(())
    }

    /// provider.rs:366-385: reports the allocator's counters and waits for the device.
    fn shutdown(&self) -> Result<()> {
        info!("Shutting down BitNet execution provider");
        let memory_info = self.allocator.get_memory_info();
        info!("  Memory allocated: {} bytes", memory_info.allocated_bytes);
        info!("  Peak memory: {} bytes", memory_info.peak_bytes);
        // SAFETY: the provider is alive as long as `self`.
        check(unsafe { sys::rbp_provider_shutdown(self.handle.raw) })
    }
}

/// provider.rs:389-391.
pub fn create_bitnet_provider() -> Result<Arc<dyn ExecutionProvider>> {
    Ok(Arc::new(BitNetExecutionProvider::new()?))
}

/// provider.rs:394-398.
pub fn create_bitnet_provider_with_config(config: BitNetProviderConfig) -> Result<Arc<dyn ExecutionProvider>> {
    Ok(Arc::new(BitNetExecutionProvider::with_config(config)?))
}

#[cfg(test)]
mod tests {
    //! The reference's own provider tests (provider.rs:400-504) restated for this provider; they
    //! need a gfx950 device.
    use super::*;
    use ronn_core::{GraphNode, Tensor, TensorLayout};
    use std::collections::HashMap;

    fn ternary() -> BitNetProviderConfig {
        BitNetProviderConfig::default()
    }

    #[test]
    fn provider_id_and_capability() -> Result<()> {
        let p = BitNetExecutionProvider::with_config(ternary())?;
        assert_eq!(p.provider_id(), ProviderId::BitNet);
        let cap = p.get_capability();
        assert_eq!(cap.performance_profile, PerformanceProfile::MemoryOptimized);
        assert!(cap.supported_ops.contains("MatMul"));
        assert!(cap.data_types.contains(&DataType::U8));
        Ok(())
    }

    #[test]
    fn known_answer_matmul() -> Result<()> {
        // inputs of the reference's test_ternary_matmul_kernel (kernels.rs:388-389); the
        // reference asserts the shape only, the values follow from its arithmetic:
        // A -> [1,-1,0,0,1,-1] scale 1.85, B -> [1,-1,0,-1,1,0] scale 1.75,
        // acc [[1,0],[-1,-1]], out = acc * 1.85 * 1.75
        let p = BitNetExecutionProvider::with_config(ternary())?;
        let node = GraphNode {
            id: 0,
            op_type: "MatMul".to_string(),
            attributes: HashMap::new(),
            inputs: vec!["a".into(), "b".into()],
            outputs: vec!["c".into()],
            name: None,
        };
        let sg = SubGraph { nodes: vec![node], edges: vec![], inputs: vec![], outputs: vec![] };
        let kernel = p.compile_subgraph(sg)?;
        let a = Tensor::from_data(vec![2.0, -1.5, 0.1, -0.05, 1.8, -2.1], vec![2, 3], DataType::F32, TensorLayout::RowMajor)?;
        let b = Tensor::from_data(vec![1.0, -2.0, 0.05, -1.5, 2.5, 0.1], vec![3, 2], DataType::F32, TensorLayout::RowMajor)?;
        let out = kernel.execute(&[a, b])?;
        assert_eq!(out.len(), 1);
        assert_eq!(out[0].shape(), vec![2, 2]);
        let bits: Vec<u32> = out[0].to_vec()?.iter().map(|v| v.to_bits()).collect();
        assert_eq!(bits, vec![0x404f3333, 0x00000000, 0xc04f3333, 0xc04f3333]); // +-3.2375
        assert_eq!(kernel.get_performance_stats().execution_count, 1);
        Ok(())
    }

    #[test]
    fn group_of_three_projections_is_one_launch() -> Result<()> {
        // q/k/v: three weight matrices, one input row; each result equals an execute() of its own
        let p = BitNetExecutionProvider::with_config(ternary())?;
        let kernel = p.create_ternary_matmul_kernel(0, 0, 0)?;
        let (k, n) = (64usize, 32usize);
        let a = Tensor::from_data((0..k).map(|i| ((i * 37 % 17) as f32 - 8.0) * 0.25).collect(), vec![1, k],
                                  DataType::F32, TensorLayout::RowMajor)?;
        let bs: Vec<Tensor> = (0..3)
            .map(|j| {
                Tensor::from_data((0..k * n).map(|i| (((i * 31 + j * 7) % 23) as f32 - 11.0) * 0.01).collect(),
                                  vec![k, n], DataType::F32, TensorLayout::RowMajor)
            })
            .collect::<Result<_>>()?;
        let pairs: Vec<(&Tensor, &Tensor)> = bs.iter().map(|b| (&a, b)).collect();
        let (outs, launches) = kernel.execute_group(&pairs)?;
        assert_eq!(launches, 1);
        for (b, got) in bs.iter().zip(&outs) {
            let single = kernel.execute(&[a.clone(), b.clone()])?;
            let want: Vec<u32> = single[0].to_vec()?.iter().map(|v| v.to_bits()).collect();
            let bits: Vec<u32> = got.to_vec()?.iter().map(|v| v.to_bits()).collect();
            assert_eq!(bits, want);
        }
        Ok(())
    }
}
