//! `CompiledKernel` for the TernaryMatMul operation on the GPU.
//!
//! Stands in for `BitNetKernel` with `BitNetOperation::TernaryMatMul`
//! (crates/ronn-providers/src/bitnet/kernels.rs:36-47, :134-178, :254-328).

use std::collections::hash_map::DefaultHasher;
use std::collections::HashMap;
use std::hash::{Hash, Hasher};
use std::os::raw::{c_int, c_void};
use std::ptr::null_mut;
use std::sync::{Arc, Mutex};
use std::time::Instant;

use anyhow::{anyhow, Result};
use ronn_bitnet_hip_sys as sys;
use ronn_core::{CompiledKernel, DataType, KernelStats, MemoryUsage, Tensor, TensorLayout};

use crate::provider::ActivationMode;

fn check(rc: c_int) -> Result<()> {
    sys::check(rc).map_err(|m| anyhow!(m))
}

/// Owns one `rbn_ctx` (one GPU, one stream).  The C side locks the context around every call,
/// which is what makes sharing it between threads sound.
pub struct HipContext {
    raw: *mut sys::rbn_ctx,
}

// SAFETY: every entry point that takes the context serialises its callers with the context's
// own lock and makes the context's device current for the calling thread.
unsafe impl Send for HipContext {}
unsafe impl Sync for HipContext {}

impl HipContext {
    pub fn new(device: i32) -> Result<Arc<Self>> {
        let mut raw = null_mut();
        // SAFETY: `raw` is a valid out-pointer.
        check(unsafe { sys::rbn_ctx_create(device as c_int, &mut raw) })?;
        Ok(Arc::new(Self { raw }))
    }

    pub fn raw(&self) -> *mut sys::rbn_ctx {
        self.raw
    }

    /// Device allocation that frees itself.
    pub fn alloc(self: &Arc<Self>, bytes: usize) -> Result<DeviceBuffer> {
        let mut p: *mut c_void = null_mut();
        // SAFETY: `p` is a valid out-pointer.
        check(unsafe { sys::rbn_malloc(self.raw, bytes, &mut p) })?;
        Ok(DeviceBuffer { ctx: Arc::clone(self), ptr: p, bytes })
    }

    pub fn upload(self: &Arc<Self>, data: &[f32]) -> Result<DeviceBuffer> {
        let buf = self.alloc(std::mem::size_of_val(data).max(4))?;
        // SAFETY: `buf` has at least `data.len() * 4` bytes.
        check(unsafe { sys::rbn_h2d(self.raw, buf.ptr, data.as_ptr().cast(), std::mem::size_of_val(data)) })?;
        Ok(buf)
    }
}

impl Drop for HipContext {
    fn drop(&mut self) {
        // SAFETY: created by rbn_ctx_create and not used after this.
        unsafe { sys::rbn_ctx_destroy(self.raw) };
    }
}

pub struct DeviceBuffer {
    ctx: Arc<HipContext>,
    ptr: *mut c_void,
    bytes: usize,
}

unsafe impl Send for DeviceBuffer {}
unsafe impl Sync for DeviceBuffer {}

impl DeviceBuffer {
    pub fn ptr<T>(&self) -> *mut T {
        self.ptr.cast()
    }
    pub fn bytes(&self) -> usize {
        self.bytes
    }
}

impl Drop for DeviceBuffer {
    fn drop(&mut self) {
        // SAFETY: allocated by rbn_malloc on this context; rbn_free waits for the stream first.
        unsafe { sys::rbn_free(self.ctx.raw, self.ptr) };
    }
}

/// A weight matrix ternarised once (`quantize_ternary`, quantization.rs:67-109) and laid out for
/// the matmul kernels.
struct TiledWeights {
    tiled: DeviceBuffer,
    scale: f32,
    k: u64,
    n: u64,
    /// Second, independent digest of the f32 data: a hit on the first key alone is not trusted.
    check: u64,
}

/// TernaryMatMul on the GPU.
pub struct HipTernaryMatMul {
    ctx: Arc<HipContext>,
    /// Ternarised weights by content key; the reference re-ternarises input 1 on every call
    /// (kernels.rs:278), here that happens once per distinct matrix.
    weights: Mutex<HashMap<u64, Arc<TiledWeights>>>,
    stats: Mutex<KernelStats>,
    memory: Mutex<MemoryUsage>,
    sum_mode: c_int,
    activation: ActivationMode,
    max_cache_bytes: usize,
}

impl HipTernaryMatMul {
    pub fn new(ctx: Arc<HipContext>, strict_reference_sum: bool, activation: ActivationMode,
               max_cache_bytes: usize) -> Self {
        Self {
            ctx,
            weights: Mutex::new(HashMap::new()),
            stats: Mutex::new(KernelStats {
                execution_count: 0,
                average_time_us: 0.0,
                min_time_us: 0.0,
                max_time_us: 0.0,
            }),
            memory: Mutex::new(MemoryUsage { peak_bytes: 0, current_bytes: 0, allocation_count: 0 }),
            sum_mode: if strict_reference_sum { sys::RBN_SUM_STRICT_SEQ } else { sys::RBN_SUM_TREE },
            activation,
            max_cache_bytes,
        }
    }

    fn digests(data: &[f32]) -> (u64, u64) {
        let mut h1 = DefaultHasher::new();
        let mut h2: u64 = 0xcbf2_9ce4_8422_2325; // FNV-1a over the bit patterns
        data.len().hash(&mut h1);
        for v in data {
            let b = v.to_bits();
            b.hash(&mut h1);
            h2 = (h2 ^ u64::from(b)).wrapping_mul(0x0000_0100_0000_01b3);
        }
        (h1.finish(), h2)
    }

    /// quantize_ternary + tiling of input 1, cached.
    fn tiled_weights(&self, b: &Tensor, k: u64, n: u64) -> Result<Arc<TiledWeights>> {
        let data = b.to_vec()?; // tensor.rs:217, row-major
        let (key, check_digest) = Self::digests(&data);
        if let Some(w) = self.weights.lock().unwrap().get(&key) {
            if w.k == k && w.n == n && w.check == check_digest {
                return Ok(Arc::clone(w));
            }
        }
        let ctx = &self.ctx;
        let d_w = ctx.upload(&data)?;
        // SAFETY: sizes come from the library's own size functions; all buffers are live until
        // the synchronous calls below have returned.
        let w = unsafe {
            let d_packed = ctx.alloc(sys::rbn_packed_capacity(k * n))?;
            let (mut scale, mut threshold, mut survivors) = (0f32, 0f32, 0u64);
            check(sys::rbn_quantize_ternary(ctx.raw(), d_w.ptr(), k * n, self.sum_mode, d_packed.ptr(),
                                            &mut scale, &mut threshold, &mut survivors))?;
            let tiled = ctx.alloc(sys::rbn_tiled_bytes(k, n))?;
            check(sys::rbn_tile_weights(ctx.raw(), d_packed.ptr(), k, n, tiled.ptr()))?;
            check(sys::rbn_sync(ctx.raw()))?;
            Arc::new(TiledWeights { tiled, scale, k, n, check: check_digest })
        };
        let mut cache = self.weights.lock().unwrap();
        let mut mem = self.memory.lock().unwrap();
        // no room: drop the cached matrices (they are rebuilt on demand) rather than grow
        if mem.current_bytes + w.tiled.bytes() > self.max_cache_bytes {
            cache.clear();
            mem.current_bytes = 0;
        }
        mem.current_bytes += w.tiled.bytes();
        mem.peak_bytes = mem.peak_bytes.max(mem.current_bytes);
        mem.allocation_count += 1;
        cache.insert(key, Arc::clone(&w));
        Ok(w)
    }

    /// kernels.rs:235-251.
    fn update_stats(&self, execution_time_us: f64) {
        let mut s = self.stats.lock().unwrap();
        s.execution_count += 1;
        if s.execution_count == 1 {
            s.min_time_us = execution_time_us;
            s.max_time_us = execution_time_us;
            s.average_time_us = execution_time_us;
        } else {
            s.min_time_us = s.min_time_us.min(execution_time_us);
            s.max_time_us = s.max_time_us.max(execution_time_us);
            let n = s.execution_count as f64;
            s.average_time_us = ((n - 1.0) * s.average_time_us + execution_time_us) / n;
        }
    }
}

impl CompiledKernel for HipTernaryMatMul {
    fn execute(&self, inputs: &[Tensor]) -> Result<Vec<Tensor>> {
        let start_time = Instant::now();
        if inputs.len() != 2 {
            return Err(anyhow!("Ternary MatMul requires exactly 2 inputs")); // kernels.rs:273
        }
        for t in inputs {
            if t.dtype() != DataType::F32 {
                // quantization.rs:68-72
                return Err(anyhow!("BitNet quantization requires FP32 input tensors"));
            }
        }
        let (a, b) = (&inputs[0], &inputs[1]);
        let (sa, sb) = (a.shape(), b.shape());
        // kernels.rs:142-152; m, n, k come from the inputs instead of the constants 64, 64, 64
        if sa.len() != 2 || sb.len() != 2 || sa[1] != sb[0] {
            return Err(anyhow!(
                "Matrix dimension mismatch: A={:?}, B={:?}, expected A=[m,k], B=[k,n]",
                sa, sb
            ));
        }
        let (m, k, n) = (sa[0] as u64, sa[1] as u64, sb[1] as u64);
        if m == 0 || k == 0 || n == 0 {
            return Err(anyhow!("Matrix dimension mismatch: A={:?}, B={:?}, expected A=[m,k], B=[k,n]", sa, sb));
        }
        let w = self.tiled_weights(b, k, n)?;
        let ctx = &self.ctx;
        let av = a.to_vec()?;
        let d_a = ctx.upload(&av)?;
        let mut out = vec![0f32; (m * n) as usize];
        // SAFETY: buffer sizes follow the header (m * rbn_act_pitch(k) int8, m f32, m int32,
        // m * n f32); rbn_d2h synchronises the stream before `out` is read.
        unsafe {
            let d_q = ctx.alloc(m as usize * sys::rbn_act_pitch(k))?;
            let d_scale = ctx.alloc(4 * m as usize)?;
            let d_rowsum = ctx.alloc(4 * m as usize)?;
            match self.activation {
                // per-token absmax int8 (no counterpart in the reference)
                ActivationMode::Int8PerToken => check(sys::rbn_act_quant_i8(
                    ctx.raw(), d_a.ptr(), m, k, d_q.ptr(), d_scale.ptr(), d_rowsum.ptr()))?,
                // the reference's own choice: quantize_ternary over the whole tensor (kernels.rs:277)
                ActivationMode::TernaryPerTensor => check(sys::rbn_act_quant_ternary(
                    ctx.raw(), d_a.ptr(), m, k, self.sum_mode, d_q.ptr(), d_scale.ptr(), d_rowsum.ptr(),
                    null_mut(), null_mut()))?,
            }
            let d_out = ctx.alloc(4 * (m * n) as usize)?;
            // kernels.rs:134-178 with the epilogue of :168
            check(sys::rbn_matmul_t2_i8(ctx.raw(), d_q.ptr(), d_scale.ptr(), d_rowsum.ptr(), w.tiled.ptr(),
                                        w.scale, m, k, n, null_mut(), d_out.ptr()))?;
            check(sys::rbn_d2h(ctx.raw(), out.as_mut_ptr().cast(), d_out.ptr::<c_void>() as *const c_void,
                               out.len() * 4))?;
        }
        let result = Tensor::from_data(out, vec![m as usize, n as usize], DataType::F32, TensorLayout::RowMajor)?;
        self.update_stats(start_time.elapsed().as_micros() as f64);
        Ok(vec![result])
    }

    fn get_memory_usage(&self) -> MemoryUsage {
        self.memory.lock().unwrap().clone()
    }

    fn get_performance_stats(&self) -> KernelStats {
        self.stats.lock().unwrap().clone()
    }
}
