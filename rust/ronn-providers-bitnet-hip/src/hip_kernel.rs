//! `CompiledKernel` for the TernaryMatMul operation on the GPU.
//!
//! Stands in for `BitNetKernel` with `BitNetOperation::TernaryMatMul`
//! (crates/ronn-providers/src/bitnet/kernels.rs:36-47, :134-178, :254-328).  The kernel object
//! itself lives behind the C ABI (`rbp_kernel`): weight cache (ternarise once, two digests,
//! least-recently-used eviction), activation quantisation, kernel choice and statistics are the
//! library's, so this file only moves tensors across the boundary.

use std::os::raw::c_int;
use std::ptr::null_mut;

use anyhow::{anyhow, Result};
use ronn_bitnet_hip_sys as sys;
use ronn_core::{CompiledKernel, DataType, KernelStats, MemoryUsage, Tensor, TensorLayout};

/// The library's message for the calling thread's last provider-level failure; for errors the
/// reference also raises it is the reference's text.
pub(crate) fn check(rc: c_int) -> Result<()> {
    sys::check_provider(rc).map_err(|m| anyhow!(m))
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

pub(crate) fn dtype_to_code(dtype: DataType) -> c_int {
    dtype_code(dtype)
}

/// One compiled BitNet kernel on the GPU.
pub struct HipKernel {
    raw: *mut sys::rbp_kernel,
}

// SAFETY: the object behind `raw` takes its own lock for the whole of every call
// (`CompiledKernel` is `Send + Sync`, types.rs:153: `execute(&self)` may run on many threads).
unsafe impl Send for HipKernel {}
unsafe impl Sync for HipKernel {}

impl HipKernel {
    /// Takes ownership of a kernel created by `rbp_provider_compile_subgraph` or
    /// `rbp_create_ternary_matmul_kernel`.
    pub(crate) fn from_raw(raw: *mut sys::rbp_kernel) -> Self {
        Self { raw }
    }

    /// Several independent TernaryMatMul nodes of one shape in one call: `pairs[i] = (A_i, B_i)`,
    /// every `A_i` `[m,k]`, every `B_i` `[k,n]`.  Result `i` is what `execute(&[A_i, B_i])`
    /// returns, bit for bit.  A graph holds such nodes side by side (the q/k/v or gate/up
    /// projections of one token; `ProviderRegistry::compile_subgraph`, registry.rs:237-266,
    /// compiles them one by one); in the decode regime the library runs up to 32 of them as one
    /// GPU launch, which is what brings a single-token matmul from a third of the memory
    /// bandwidth towards all of it.  Returns the results and the number of launches issued.
    pub fn execute_group(&self, pairs: &[(&Tensor, &Tensor)]) -> Result<(Vec<Tensor>, usize)> {
        if pairs.is_empty() {
            return Err(anyhow!("Ternary MatMul group requires pairs of inputs (A_i, B_i)"));
        }
        for (a, b) in pairs {
            if a.dtype() != DataType::F32 || b.dtype() != DataType::F32 {
                // quantization.rs:68-72
                return Err(anyhow!("BitNet quantization requires FP32 input tensors"));
            }
        }
        let (sa, sb) = (pairs[0].0.shape(), pairs[0].1.shape());
        if sa.len() != 2 || sb.len() != 2 {
            return Err(anyhow!("Matrix dimension mismatch: A={:?}, B={:?}, expected A=[m,k], B=[k,n]", sa, sb));
        }
        // the C entry point takes one shape for the whole group
        for (i, (a, b)) in pairs.iter().enumerate().skip(1) {
            if a.shape() != sa || b.shape() != sb {
                return Err(anyhow!(
                    "Ternary MatMul group: node {} has A={:?}, B={:?}, the group's shape is A={:?}, B={:?}",
                    i, a.shape(), b.shape(), sa, sb
                ));
            }
        }
        let a_data: Vec<Vec<f32>> = pairs.iter().map(|(a, _)| a.to_vec()).collect::<Result<_>>()?;
        let b_data: Vec<Vec<f32>> = pairs.iter().map(|(_, b)| b.to_vec()).collect::<Result<_>>()?;
        let (m, n) = (sa[0], sb[1]);
        let mut outs: Vec<Vec<f32>> = pairs.iter().map(|_| vec![0f32; (m * n).max(1)]).collect();
        let pa: Vec<*const f32> = a_data.iter().map(|v| v.as_ptr()).collect();
        let pb: Vec<*const f32> = b_data.iter().map(|v| v.as_ptr()).collect();
        let po: Vec<*mut f32> = outs.iter_mut().map(|v| v.as_mut_ptr()).collect();
        let shape_a = [sa[0] as u64, sa[1] as u64];
        let shape_b = [sb[0] as u64, sb[1] as u64];
        let mut launches: c_int = 0;
        // SAFETY: every pointer array has `pairs.len()` live entries; each input holds the number
        // of elements its shape says (Tensor::to_vec); each output has `out_capacity_each` elements.
        check(unsafe {
            sys::rbp_kernel_execute_group(
                self.raw,
                pairs.len() as c_int,
                pa.as_ptr(),
                pb.as_ptr(),
                shape_a.as_ptr(),
                shape_b.as_ptr(),
                po.as_ptr(),
                (m * n).max(1) as u64,
                &mut launches,
            )
        })?;
        let mut results = Vec::with_capacity(outs.len());
        for mut o in outs {
            o.truncate(m * n);
            results.push(Tensor::from_data(o, vec![m, n], DataType::F32, TensorLayout::RowMajor)?);
        }
        Ok((results, launches as usize))
    }
}

impl Drop for HipKernel {
    fn drop(&mut self) {
        // SAFETY: created by the library, not used after this.
        unsafe { sys::rbp_kernel_destroy(self.raw) };
    }
}

impl CompiledKernel for HipKernel {
    /// kernels.rs:254-319.  Input checks, error texts ("Ternary MatMul requires exactly 2
    /// inputs", "Matrix dimension mismatch: ...", "BitNet quantization requires FP32 input
    /// tensors") and the arithmetic are the library's; m, n, k come from the inputs.
    fn execute(&self, inputs: &[Tensor]) -> Result<Vec<Tensor>> {
        let data: Vec<Vec<f32>> = inputs
            .iter()
            .map(|t| if t.dtype() == DataType::F32 { t.to_vec() } else { Ok(Vec::new()) })
            .collect::<Result<_>>()?;
        let shapes: Vec<Vec<u64>> = inputs.iter().map(|t| t.shape().iter().map(|&d| d as u64).collect()).collect();
        let data_p: Vec<*const f32> = data.iter().map(|v| v.as_ptr()).collect();
        let shape_p: Vec<*const u64> = shapes.iter().map(|v| v.as_ptr()).collect();
        let ndims: Vec<c_int> = shapes.iter().map(|v| v.len() as c_int).collect();
        let dtypes: Vec<c_int> = inputs.iter().map(|t| dtype_code(t.dtype())).collect();
        // [m, n] of a well-formed call; anything else is rejected by the library before it writes
        let capacity = match (shapes.first(), shapes.get(1)) {
            (Some(a), Some(b)) if a.len() == 2 && b.len() == 2 => (a[0] * b[1]).max(1) as usize,
            _ => 1,
        };
        let mut out = vec![0f32; capacity];
        let mut out_shape = [0u64; 2];
        // SAFETY: the arrays have `inputs.len()` live entries; a non-F32 tensor is refused on its
        // dtype code before its (empty) data is looked at; `out` has `capacity` elements.
        check(unsafe {
            sys::rbp_kernel_execute(
                self.raw,
                inputs.len() as c_int,
                data_p.as_ptr(),
                shape_p.as_ptr(),
                ndims.as_ptr(),
                dtypes.as_ptr(),
                out.as_mut_ptr(),
                capacity as u64,
                out_shape.as_mut_ptr(),
            )
        })?;
        let (m, n) = (out_shape[0] as usize, out_shape[1] as usize);
        out.truncate(m * n);
        Ok(vec![Tensor::from_data(out, vec![m, n], DataType::F32, TensorLayout::RowMajor)?])
    }

    /// kernels.rs:321-323; here the bytes of cached, ternarised weights.
    fn get_memory_usage(&self) -> MemoryUsage {
        let (mut peak, mut current, mut allocations) = (0u64, 0u64, 0u64);
        // SAFETY: valid out-pointers.
        let _ = unsafe { sys::rbp_kernel_memory_usage(self.raw, &mut peak, &mut current, &mut allocations) };
        MemoryUsage {
            peak_bytes: peak as usize,
            current_bytes: current as usize,
            allocation_count: allocations as usize,
        }
    }

    /// kernels.rs:325-327; really updated (the reference measures and drops, :313-316).
    fn get_performance_stats(&self) -> KernelStats {
        let (mut count, mut avg, mut lo, mut hi) = (0u64, 0f64, 0f64, 0f64);
        // SAFETY: valid out-pointers.
        let _ = unsafe { sys::rbp_kernel_stats(self.raw, &mut count, &mut avg, &mut lo, &mut hi) };
        KernelStats { execution_count: count, average_time_us: avg, min_time_us: lo, max_time_us: hi }
    }
}

/// Keeps `null_mut` in one place for the callers that create kernels.
pub(crate) fn null_kernel() -> *mut sys::rbp_kernel {
    null_mut()
}
