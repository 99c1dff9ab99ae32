//! `ProviderId::BitNet` on an AMD MI355X.
//!
//! Drop-in for `crates/ronn-providers/src/bitnet/` of the reference: the same public names
//! (`BitNetExecutionProvider`, `BitNetProviderConfig`, `QuantizationMethod`,
//! `create_bitnet_provider`, `create_bitnet_provider_with_config`), the same traits
//! (`ExecutionProvider`, `CompiledKernel`, `TensorAllocator`, crates/ronn-core/src/types.rs:153-303),
//! the same error texts; the arithmetic runs in hand-written gfx950 kernels behind
//! `ronn-bitnet-hip-sys`.  There is no CPU fallback: without a gfx950 device
//! `create_bitnet_provider` returns the library's "no HIP device visible" error.
//!
//! Deliberate differences from the reference's provider, each stated where it occurs:
//! kernels take m, n, k from their inputs (the reference hard-codes 64^3, provider.rs:157-159);
//! the weight operand is ternarised once and cached (the reference redoes it on every call,
//! kernels.rs:278); `KernelStats` are really updated (kernels.rs:313-316 drops them); the binary
//! (XNOR) half of the reference is not implemented and says so.

pub mod hip_kernel;
pub mod provider;

pub use hip_kernel::HipKernel;
pub use provider::{
    create_bitnet_provider, create_bitnet_provider_with_config, ActivationMode, BitNetExecutionProvider,
    BitNetHipAllocator, BitNetMemoryStats, BitNetProviderConfig, QuantizationMethod,
};
