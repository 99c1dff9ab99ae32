//! `ExecutionProvider` with `ProviderId::BitNet` on an MI355X.
//!
//! Stands in for `BitNetExecutionProvider` (crates/ronn-providers/src/bitnet/provider.rs:25-398)
//! and `BitNetMemoryAllocator` (bitnet/allocator.rs:15-149).

use std::collections::HashSet;
use std::os::raw::{c_int, c_void};
use std::ptr::null_mut;
use std::sync::atomic::{AtomicUsize, Ordering};
use std::sync::Arc;

use anyhow::{anyhow, Result};
use ronn_bitnet_hip_sys as sys;
use ronn_core::{
    CompiledKernel, DataType, ExecutionProvider, GraphNode, MemoryInfo, MemoryType, OperatorSpec,
    OptimizationLevel, PerformanceProfile, ProviderCapability, ProviderConfig, ProviderId,
    ResourceRequirements, SubGraph, TensorAllocator, TensorBuffer,
};
use tracing::{debug, info, warn};

use crate::hip_kernel::{HipContext, HipTernaryMatMul};

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

impl Default for BitNetProviderConfig {
    fn default() -> Self {
        Self {
            // the reference defaults to Binary (provider.rs:60); only the ternary half exists here
            quantization_method: QuantizationMethod::Ternary,
            enable_kernel_caching: true,
            max_cache_size: 64 * 1024 * 1024,
            enable_mixed_precision: true,
            memory_optimization_level: 2,
            enable_simd: true,
            activation: ActivationMode::TernaryPerTensor,
            strict_reference_sum: true,
            device: 0,
        }
    }
}

/// Device-memory `TensorAllocator` with the reference's size and alignment rules
/// (allocator.rs:39-75): U8 = 2-bit ternary, 4 elements per byte; Bool = 1 bit per element.
pub struct BitNetHipAllocator {
    ctx: Arc<HipContext>,
    allocated_bytes: AtomicUsize,
    peak_bytes: AtomicUsize,
    total_bytes: usize,
}

fn dtype_code(dtype: DataType) -> c_int {
    match dtype {
        DataType::F32 => sys::RBN_DT_F32,
        DataType::F16 => sys::RBN_DT_F16,
        DataType::BF16 => sys::RBN_DT_BF16,
        DataType::I8 => sys::RBN_DT_I8,
        DataType::I32 => sys::RBN_DT_I32,
        DataType::I64 => sys::RBN_DT_I64,
        DataType::U8 => sys::RBN_DT_U8,
        DataType::U32 => sys::RBN_DT_U32,
        DataType::Bool => sys::RBN_DT_BOOL,
        DataType::F64 => sys::RBN_DT_F64,
    }
}

impl BitNetHipAllocator {
    pub fn new(ctx: Arc<HipContext>) -> Result<Self> {
        // SAFETY: plain-old-data out-parameter.
        let mut info: sys::rbn_device_info = unsafe { std::mem::zeroed() };
        sys::check(unsafe { sys::rbn_get_device_info(ctx.raw(), &mut info) }).map_err(|m| anyhow!(m))?;
        Ok(Self {
            ctx,
            allocated_bytes: AtomicUsize::new(0),
            peak_bytes: AtomicUsize::new(0),
            total_bytes: info.hbm_bytes as usize,
        })
    }
}

impl TensorAllocator for BitNetHipAllocator {
    fn allocate(&self, shape: &[usize], dtype: DataType) -> Result<TensorBuffer> {
        let element_count: usize = shape.iter().product();
        // SAFETY: pure functions of their arguments.
        let size = unsafe { sys::rbn_tensor_bytes(element_count as u64, dtype_code(dtype)) };
        if size < 0 {
            // allocator.rs:61-64
            return Err(anyhow!("Unsupported data type for BitNet allocator: {:?}", dtype));
        }
        let size = size as usize;
        let alignment = unsafe { sys::rbn_tensor_alignment(dtype_code(dtype)) };
        let mut p: *mut c_void = null_mut();
        // SAFETY: valid out-pointer; device memory comes back 256-byte aligned.
        sys::check(unsafe { sys::rbn_malloc(self.ctx.raw(), size, &mut p) })
            .map_err(|m| anyhow!("Memory allocation failed for {} bytes: {}", size, m))?;
        let now = self.allocated_bytes.fetch_add(size, Ordering::Relaxed) + size;
        self.peak_bytes.fetch_max(now, Ordering::Relaxed);
        Ok(TensorBuffer { ptr: p.cast(), size, alignment, memory_type: MemoryType::DeviceMemory })
    }

    fn deallocate(&self, buffer: TensorBuffer) -> Result<()> {
        // SAFETY: `buffer.ptr` came from `allocate` above.
        sys::check(unsafe { sys::rbn_free(self.ctx.raw(), buffer.ptr.cast()) }).map_err(|m| anyhow!(m))?;
        self.allocated_bytes.fetch_sub(buffer.size, Ordering::Relaxed);
        Ok(())
    }

    fn get_memory_info(&self) -> MemoryInfo {
        MemoryInfo {
            total_bytes: self.total_bytes,
            allocated_bytes: self.allocated_bytes.load(Ordering::Relaxed),
            peak_bytes: self.peak_bytes.load(Ordering::Relaxed),
        }
    }
}

/// BitNet execution provider backed by the gfx950 kernels.
pub struct BitNetExecutionProvider {
    config: BitNetProviderConfig,
    ctx: Arc<HipContext>,
    allocator: Arc<dyn TensorAllocator>,
    supported_ops: HashSet<String>,
}

impl BitNetExecutionProvider {
    pub fn new() -> Result<Self> {
        Self::with_config(BitNetProviderConfig::default())
    }

    /// provider.rs:77-114: resources and the supported-operation set.
    pub fn with_config(config: BitNetProviderConfig) -> Result<Self> {
        info!("Creating BitNet execution provider with method: {:?}", config.quantization_method);
        let ctx = HipContext::new(config.device)?;
        let allocator: Arc<dyn TensorAllocator> = Arc::new(BitNetHipAllocator::new(Arc::clone(&ctx))?);
        // provider.rs:87-99: the same twelve names, so that can_handle answers as before; the
        // operations outside the ternary matmul fail at compile_subgraph with a message that says so
        let supported_ops: HashSet<String> = [
            "MatMul", "Gemm", "Conv", "Add", "Sub", "Mul", "And", "Or", "Xor", "BatchNormalization", "ReLU",
            "Sigmoid",
        ]
        .iter()
        .map(|s| s.to_string())
        .collect();
        info!("BitNet provider supports {} operations", supported_ops.len());
        Ok(Self { config, ctx, allocator, supported_ops })
    }

    pub fn get_config(&self) -> &BitNetProviderConfig {
        &self.config
    }

    pub fn supports_operation(&self, op_type: &str) -> bool {
        self.supported_ops.contains(op_type)
    }

    /// provider.rs:132-150, the same constants.
    pub fn estimate_speedup(&self, op_spec: &OperatorSpec) -> f32 {
        match op_spec.op_type.as_str() {
            "MatMul" | "Gemm" => match self.config.quantization_method {
                QuantizationMethod::Binary => 64.0,
                QuantizationMethod::Ternary => 32.0,
                QuantizationMethod::AsymmetricBinary { .. } => 48.0,
            },
            "Conv" => match self.config.quantization_method {
                QuantizationMethod::Binary => 32.0,
                QuantizationMethod::Ternary => 24.0,
                QuantizationMethod::AsymmetricBinary { .. } => 28.0,
            },
            "Add" | "Sub" | "Mul" => 16.0,
            "And" | "Or" | "Xor" => 128.0,
            _ => 4.0,
        }
    }

    /// provider.rs:153-210.  MatMul / Gemm with the ternary method get the GPU kernel, which
    /// takes m, n, k from its inputs (the reference fixes them at 64).
    fn create_kernel_for_operation(&self, node: &GraphNode) -> Result<Box<dyn CompiledKernel>> {
        match node.op_type.as_str() {
            "MatMul" | "Gemm" => match self.config.quantization_method {
                QuantizationMethod::Ternary => Ok(Box::new(HipTernaryMatMul::new(
                    Arc::clone(&self.ctx),
                    self.config.strict_reference_sum,
                    self.config.activation,
                    self.config.max_cache_size,
                ))),
                _ => Err(anyhow!(
                    "Binary (XNOR) kernels are not part of the MI355X BitNet provider: configure quantization_method = ternary"
                )),
            },
            "And" | "Or" | "Xor" | "Add" | "Sub" | "Mul" | "Conv" | "ReLU" | "BatchNormalization" => Err(anyhow!(
                "Operation {} runs on binary kernels, which are not part of the MI355X BitNet provider",
                node.op_type
            )),
            _ => Err(anyhow!("Unsupported operation for BitNet: {}", node.op_type)), // provider.rs:205-208
        }
    }
}

impl ExecutionProvider for BitNetExecutionProvider {
    fn provider_id(&self) -> ProviderId {
        ProviderId::BitNet
    }

    /// provider.rs:250-271 with the memory type of this implementation.
    fn get_capability(&self) -> ProviderCapability {
        ProviderCapability {
            supported_ops: self.supported_ops.clone(),
            data_types: vec![DataType::Bool, DataType::U8, DataType::F32, DataType::F16],
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

    /// provider.rs:280-310.  The reference's cache lookup can only fail ("Kernel caching not
    /// fully implemented", :289-293, on a map that is never filled); there is no such map here:
    /// what is worth caching - the ternarised weights - is cached inside the kernel.
    fn compile_subgraph(&self, subgraph: SubGraph) -> Result<Box<dyn CompiledKernel>> {
        debug!("Compiling BitNet subgraph with {} nodes", subgraph.nodes.len());
        if subgraph.nodes.len() != 1 {
            return Err(anyhow!("BitNet provider currently supports only single-node subgraphs"));
        }
        let node = &subgraph.nodes[0];
        let kernel = self.create_kernel_for_operation(node)?;
        info!("Successfully compiled BitNet kernel for {}", node.op_type);
        Ok(kernel)
    }

    fn get_allocator(&self) -> Arc<dyn TensorAllocator> {
        Arc::clone(&self.allocator)
    }

    /// provider.rs:316-364.  `custom_options` are applied at every optimisation level (the
    /// reference parses them only under `Custom`, although its own test sets them under
    /// `Aggressive`, provider.rs:479-500); two keys are new: `activation` = ternary | int8 and
    /// `strict_reference_sum` = true | false.
    fn configure(&mut self, config: ProviderConfig) -> Result<()> {
        if let Some(memory_limit) = config.memory_limit {
            self.config.max_cache_size = (memory_limit / 4).min(128 * 1024 * 1024);
        }
        match config.optimization_level {
            OptimizationLevel::None => {
                self.config.memory_optimization_level = 0;
                self.config.enable_simd = false;
            }
            OptimizationLevel::Basic => {
                self.config.memory_optimization_level = 1;
                self.config.enable_simd = true;
            }
            OptimizationLevel::Aggressive => {
                self.config.memory_optimization_level = 2;
                self.config.enable_simd = true;
                self.config.enable_mixed_precision = true;
            }
            OptimizationLevel::Custom => {}
        }
        for (key, value) in &config.custom_options {
            match key.as_str() {
                "quantization_method" => {
                    self.config.quantization_method = match value.as_str() {
                        "binary" => QuantizationMethod::Binary,
                        "ternary" => QuantizationMethod::Ternary,
                        _ => QuantizationMethod::Binary,
                    };
                }
                "enable_mixed_precision" => {
                    self.config.enable_mixed_precision = value.parse().unwrap_or(true);
                }
                "enable_simd" => {
                    self.config.enable_simd = value.parse().unwrap_or(true);
                }
                "activation" => {
                    self.config.activation = match value.as_str() {
                        "int8" => ActivationMode::Int8PerToken,
                        _ => ActivationMode::TernaryPerTensor,
                    };
                }
                "strict_reference_sum" => {
                    self.config.strict_reference_sum = value.parse().unwrap_or(true);
                }
                _ => warn!("Unknown BitNet config option: {}", key),
            }
        }
        info!("BitNet provider reconfigured with optimization level: {:?}", config.optimization_level);
        Ok(())
    }

    /// provider.rs:366-385.
    fn shutdown(&self) -> Result<()> {
        info!("Shutting down BitNet execution provider");
        let memory_info = self.allocator.get_memory_info();
        info!("  Memory allocated: {} bytes", memory_info.allocated_bytes);
        info!("  Peak memory: {} bytes", memory_info.peak_bytes);
        // SAFETY: the context is alive as long as `self`.
        sys::check(unsafe { sys::rbn_sync(self.ctx.raw()) }).map_err(|m| anyhow!(m))
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
    use ronn_core::{Tensor, TensorLayout};
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
}
