"""The provider-level drop-in on a real MI355X.

These mirror the reference's own #[cfg(test)] modules, with values checked where the
reference only checks shapes:
  crates/ronn-providers/src/bitnet/quantization.rs:294-363
  crates/ronn-providers/src/bitnet/kernels.rs:357-434
  crates/ronn-providers/src/bitnet/provider.rs:400-504
  crates/ronn-providers/src/bitnet/allocator.rs:213-293
"""
import threading

import numpy as np
import pytest

from oracle import oracle as O
from ronn_amd.bitnet import (BitNetExecutionProvider, BitNetProviderConfig, DataType, Error,
                             GraphNode, OperatorSpec, OptimizationLevel, PerformanceProfile,
                             ProviderConfig, ProviderId, QuantizationMethod, SubGraph, Tensor,
                             create_bitnet_provider, create_bitnet_provider_with_config)
from ronn_amd.device import synth_normal
from util import same_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def provider():
    return create_bitnet_provider()


def matmul_subgraph(op="MatMul", nodes=1):
    return SubGraph(nodes=[GraphNode(id=i, op_type=op, inputs=["A", "B"], outputs=["C"],
                                     name="test_matmul") for i in range(nodes)],
                    inputs=["A", "B"], outputs=["C"])


# ---- provider.rs tests ------------------------------------------------------------------------

def test_bitnet_provider_creation(provider):                      # provider.rs:406-415
    assert provider.provider_id() == ProviderId.BitNet
    assert provider.supports_operation("MatMul")
    assert provider.supports_operation("Conv")
    assert not provider.supports_operation("LSTM")


def test_memory_stats_start_empty(provider):                      # provider.rs:121-123, allocator.rs:168-175
    assert provider.get_memory_stats() == {"binary_tensor_count": 0, "ternary_tensor_count": 0,
                                           "memory_saved_bytes": 0, "average_compression_ratio": 1.0}


def test_provider_capabilities(provider):                         # provider.rs:418-432
    cap = provider.get_capability()
    assert "MatMul" in cap["supported_ops"] and "And" in cap["supported_ops"]
    assert len(cap["supported_ops"]) == 12
    assert DataType.Bool in cap["data_types"] and DataType.F32 in cap["data_types"]
    assert cap["performance_profile"] == PerformanceProfile.MemoryOptimized
    assert provider.can_handle([OperatorSpec("MatMul"), OperatorSpec("LSTM"), OperatorSpec("Gemm")]) \
        == [True, False, True]


def test_speedup_estimation():                                    # provider.rs:435-452
    p = create_bitnet_provider_with_config(
        BitNetProviderConfig(quantization_method=QuantizationMethod.Binary))
    assert p.estimate_speedup(OperatorSpec("MatMul", [DataType.F32, DataType.F32], [DataType.F32])) == 64.0
    t = create_bitnet_provider()
    assert t.estimate_speedup(OperatorSpec("MatMul")) == 32.0
    assert t.estimate_speedup(OperatorSpec("Conv")) == 24.0
    assert t.estimate_speedup(OperatorSpec("Xor")) == 128.0
    assert t.estimate_speedup(OperatorSpec("Softmax")) == 4.0


def test_subgraph_compilation(provider):                          # provider.rs:455-476
    kernel = provider.compile_subgraph(matmul_subgraph())
    assert kernel.get_performance_stats().execution_count == 0
    assert kernel.get_memory_usage().current_bytes == 0
    with pytest.raises(Error, match="supports only single-node subgraphs"):   # provider.rs:297-301
        provider.compile_subgraph(matmul_subgraph(nodes=2))
    with pytest.raises(Error, match="Unsupported operation for BitNet: LSTM"):  # provider.rs:205-208
        provider.compile_subgraph(matmul_subgraph(op="LSTM"))
    with pytest.raises(Error, match="outside this build"):
        provider.compile_subgraph(matmul_subgraph(op="Conv"))


def test_provider_configuration():                                # provider.rs:479-503
    p = create_bitnet_provider_with_config(
        BitNetProviderConfig(quantization_method=QuantizationMethod.Binary))
    p.configure(ProviderConfig(memory_limit=256 * 1024 * 1024,
                               optimization_level=OptimizationLevel.Aggressive,
                               custom_options={"quantization_method": "ternary",
                                               "enable_mixed_precision": "false"}))
    cfg = p.config
    assert cfg.quantization_method == QuantizationMethod.Ternary
    assert not cfg.enable_mixed_precision
    assert cfg.max_cache_size == 64 * 1024 * 1024          # min(limit / 4, 128 MiB), provider.rs:318-320
    assert cfg.memory_optimization_level == 2 and cfg.enable_simd
    p.configure(ProviderConfig(optimization_level=OptimizationLevel.NONE))
    assert p.config.memory_optimization_level == 0 and not p.config.enable_simd
    p.configure(ProviderConfig(optimization_level=OptimizationLevel.Custom,
                               custom_options={"activation": "int8", "strict_reference_sum": "false",
                                               "quantization_method": "nonsense"}))
    cfg = p.config
    assert cfg.activation == "int8" and not cfg.strict_reference_sum
    assert cfg.quantization_method == QuantizationMethod.Binary   # unknown value -> Binary, :344
    p.shutdown()


def test_binary_method_is_reported_as_out_of_scope():
    p = create_bitnet_provider_with_config(
        BitNetProviderConfig(quantization_method=QuantizationMethod.Binary))
    with pytest.raises(Error, match="Binary quantization is outside this build"):
        p.compile_subgraph(matmul_subgraph())


# ---- kernels.rs tests ---------------------------------------------------------------------------

def test_ternary_matmul_kernel(provider):                         # kernels.rs:384-400
    kernel = provider.create_ternary_matmul_kernel(2, 2, 3)
    a = Tensor.from_data([2.0, -1.5, 0.1, -0.05, 1.8, -2.1], [2, 3])
    b = Tensor.from_data([1.0, -2.0, 0.05, -1.5, 2.5, 0.1], [3, 2])
    results = kernel.execute([a, b])
    assert len(results) == 1 and results[0].shape() == [2, 2]
    want, _ = O.execute_ternary(a.numpy(), b.numpy())
    assert same_bits(results[0].numpy(), want)
    assert np.allclose(results[0].numpy(), [[3.2375, 0.0], [-3.2375, -3.2375]])
    st = kernel.get_performance_stats()
    assert st.execution_count == 1 and st.min_time_us == st.max_time_us == st.average_time_us > 0


def test_kernel_input_errors(provider):
    kernel = provider.create_ternary_matmul_kernel(2, 2, 3)
    a = Tensor.from_data(np.ones(6), [2, 3])
    b = Tensor.from_data(np.ones(6), [3, 2])
    with pytest.raises(Error, match="Ternary MatMul requires exactly 2 inputs"):   # kernels.rs:272-274
        kernel.execute([a])
    with pytest.raises(Error, match="Ternary MatMul requires exactly 2 inputs"):
        kernel.execute([a, b, b])
    with pytest.raises(Error, match=r"Matrix dimension mismatch: A=\[3, 2\], B=\[2, 3\], "
                                    r"expected A=\[2,3\], B=\[3,2\]"):            # kernels.rs:142-152
        kernel.execute([b, a])
    with pytest.raises(Error, match="BitNet quantization requires FP32 input tensors"):  # quantization.rs:68-72
        kernel.execute([Tensor.from_data(np.ones(6), [2, 3], DataType.I32), b])
    compiled = provider.compile_subgraph(matmul_subgraph())
    with pytest.raises(Error, match="Matrix dimension mismatch"):
        compiled.execute([a, a])       # inner dimensions differ


@pytest.mark.parametrize("m,k,n", [(64, 64, 64), (1, 2048, 2048), (4, 300, 77), (40, 256, 192)])
def test_compiled_kernel_matches_reference_execute(provider, m, k, n):
    # the provider path end to end (compile_subgraph -> execute) against the reference algorithm
    kernel = provider.compile_subgraph(matmul_subgraph("Gemm"))
    a = synth_normal(100 + m, 1.0, (m, k))
    b = synth_normal(200 + n, 0.02, (k, n))
    out = kernel.execute([Tensor.from_data(a, [m, k]), Tensor.from_data(b, [k, n])])[0]
    want, _ = O.execute_ternary(a, b)
    assert out.shape() == [m, n] and same_bits(out.numpy(), want)


def test_weight_cache_and_stats(provider):
    kernel = provider.compile_subgraph(matmul_subgraph())
    b = synth_normal(7, 0.02, (256, 128))
    tb = Tensor.from_data(b, [256, 128])
    outs = []
    for i in range(3):
        a = synth_normal(20 + i, 1.0, (2, 256))
        outs.append((a, kernel.execute([Tensor.from_data(a, [2, 256]), tb])[0].numpy()))
    for a, got in outs:
        assert same_bits(got, O.execute_ternary(a, b)[0])
    mem = kernel.get_memory_usage()
    assert mem.allocation_count == 1 and mem.current_bytes == 256 * 128 // 4   # one cached weight
    b2 = b.copy()
    b2[3, 5] = 1.0                                                            # different content
    a = outs[0][0]
    got = kernel.execute([Tensor.from_data(a, [2, 256]), Tensor.from_data(b2, [256, 128])])[0].numpy()
    assert same_bits(got, O.execute_ternary(a, b2)[0])
    assert kernel.get_memory_usage().allocation_count == 2
    st = kernel.get_performance_stats()
    assert st.execution_count == 4 and st.min_time_us <= st.average_time_us <= st.max_time_us


def test_weight_cache_evicts_least_recently_used():
    # room for two 256 x 128 matrices (8 KiB each, tiled): a third evicts the one not used for longest,
    # and every product is still right
    p = create_bitnet_provider_with_config(BitNetProviderConfig(max_cache_size=2 * 256 * 128 // 4))
    kernel = p.compile_subgraph(matmul_subgraph())
    a = synth_normal(61, 1.0, (2, 256))
    ta = Tensor.from_data(a, [2, 256])
    mats = [synth_normal(70 + i, 0.02, (256, 128)) for i in range(3)]

    def run(i):
        got = kernel.execute([ta, Tensor.from_data(mats[i], [256, 128])])[0].numpy()
        assert same_bits(got, O.execute_ternary(a, mats[i])[0]), i
        return kernel.get_memory_usage()

    assert run(0).allocation_count == 1
    assert run(1).allocation_count == 2
    assert run(0).allocation_count == 2                      # hit
    m = run(2)                                               # evicts matrix 1, not matrix 0
    assert m.allocation_count == 3 and m.current_bytes == 2 * 256 * 128 // 4
    assert run(0).allocation_count == 3                      # still cached
    assert run(1).allocation_count == 4                      # was evicted: rebuilt


def _pairs(a_list, b_list):
    out = []
    for a, b in zip(a_list, b_list):
        out += [Tensor.from_data(a, list(a.shape)), Tensor.from_data(b, list(b.shape))]
    return out


@pytest.mark.parametrize("m,k,n,count,shared_a", [(1, 512, 384, 3, True), (1, 2048, 1000, 2, True),
                                                  (2, 300, 77, 5, False), (1, 256, 128, 40, False),
                                                  (8, 256, 192, 2, False), (48, 128, 64, 3, True)])
def test_execute_group_is_every_node_on_its_own(provider, m, k, n, count, shared_a):
    # independent MatMul nodes of one shape (q/k/v share their input, other groups do not): each
    # result against the reference algorithm and against an execute() of its own; in the decode
    # regime the whole group is one launch (two beyond 32 nodes), other shapes launch per node
    kernel = provider.compile_subgraph(matmul_subgraph())
    a0 = synth_normal(900 + m, 1.0, (m, k))
    a_list = [a0 if shared_a else synth_normal(910 + i, 1.0 + 0.1 * i, (m, k)) for i in range(count)]
    b_list = [synth_normal(950 + i + n, 0.02, (k, n)) for i in range(count)]
    outs = kernel.execute_group(_pairs(a_list, b_list))
    decode = m <= 2
    assert kernel.last_group_launches == ((count + 31) // 32 if decode else count)
    assert len(outs) == count
    for i, (a, b, got) in enumerate(zip(a_list, b_list, outs)):
        assert got.shape() == [m, n]
        assert same_bits(got.numpy(), O.execute_ternary(a, b)[0]), i
        if i < 4:
            single = kernel.execute([Tensor.from_data(a, [m, k]), Tensor.from_data(b, [k, n])])[0]
            assert same_bits(got.numpy(), single.numpy()), i
    assert kernel.get_performance_stats().execution_count == count + min(count, 4)


def test_execute_group_int8_activations_and_a_cache_smaller_than_the_group():
    # room for one 256 x 128 matrix only: the group's other matrices live for the call and are
    # freed afterwards, the cached one is not evicted under the group's feet
    p = create_bitnet_provider_with_config(BitNetProviderConfig(activation="int8", max_cache_size=256 * 128 // 4))
    kernel = p.compile_subgraph(matmul_subgraph())
    a_list = [synth_normal(1000 + i, 1.0, (1, 256)) for i in range(4)]
    b_list = [synth_normal(1100 + i, 0.02, (256, 128)) for i in range(4)]
    for _ in range(2):
        outs = kernel.execute_group(_pairs(a_list, b_list))
        assert kernel.last_group_launches == 1
        for i, (a, b, got) in enumerate(zip(a_list, b_list, outs)):
            q, sc, _ = O.act_quant_i8(a)
            want, _ = O.matmul_i8_ternary(q, sc, O.quantize_ternary(b))
            assert same_bits(got.numpy(), want), i
    assert kernel.get_memory_usage().current_bytes == 256 * 128 // 4


def test_execute_group_input_errors(provider):
    kernel = provider.compile_subgraph(matmul_subgraph())
    a = Tensor.from_data(np.ones((1, 64), np.float32), [1, 64])
    b = Tensor.from_data(np.ones((64, 32), np.float32), [64, 32])
    with pytest.raises(Error, match="requires pairs of inputs"):
        kernel.execute_group([a, b, a])
    with pytest.raises(Error, match="requires pairs of inputs"):
        kernel.execute_group([])
    with pytest.raises(Error, match="node 1 has"):
        kernel.execute_group([a, b, a, Tensor.from_data(np.ones((64, 16), np.float32), [64, 16])])
    with pytest.raises(Error, match="Matrix dimension mismatch"):
        kernel.execute_group([b, b])
    with pytest.raises(Error, match="requires FP32 input tensors"):
        kernel.execute_group([a, Tensor.from_data(np.ones((64, 32), np.float32), [64, 32], DataType.F16)])
    sized = provider.create_ternary_matmul_kernel(1, 32, 64)
    assert len(sized.execute_group([a, b, a, b])) == 2
    with pytest.raises(Error, match="Matrix dimension mismatch"):
        provider.create_ternary_matmul_kernel(2, 32, 64).execute_group([a, b])


def test_int8_activation_mode():
    p = create_bitnet_provider_with_config(BitNetProviderConfig(activation="int8"))
    kernel = p.compile_subgraph(matmul_subgraph())
    a = synth_normal(31, 1.0, (3, 512))
    b = synth_normal(32, 0.02, (512, 96))
    got = kernel.execute([Tensor.from_data(a, [3, 512]), Tensor.from_data(b, [512, 96])])[0].numpy()
    q, s, _ = O.act_quant_i8(a)
    want, _ = O.matmul_i8_ternary(q, s, O.quantize_ternary(b))
    assert same_bits(got, want)


def test_kernel_is_usable_from_several_threads(provider):
    # CompiledKernel is Send + Sync in the reference (types.rs:153)
    kernel = provider.compile_subgraph(matmul_subgraph())
    b = synth_normal(9, 0.02, (128, 64))
    want = {}
    for i in range(4):
        a = synth_normal(50 + i, 1.0, (2, 128))
        want[i] = (a, O.execute_ternary(a, b)[0])
    errors = []

    def work(i):
        try:
            for _ in range(5):
                got = kernel.execute([Tensor.from_data(want[i][0], [2, 128]),
                                      Tensor.from_data(b, [128, 64])])[0].numpy()
                if not same_bits(got, want[i][1]):
                    errors.append("mismatch in thread %d" % i)
        except Exception as e:  # noqa: BLE001
            errors.append(repr(e))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors
    assert kernel.get_performance_stats().execution_count == 20


# ---- quantization.rs tests ------------------------------------------------------------------------

def test_ternary_quantization_roundtrip(provider):                # quantization.rs:315-328
    data = [2.0, -1.5, 0.1, -0.05, 1.8, -2.1, 0.02, -0.01]
    tensor = Tensor.from_data(data, [2, 4])
    quantizer = provider.quantizer()
    tt = quantizer.quantize_ternary(tensor)
    deq = quantizer.dequantize_ternary(tt)
    assert deq.shape() == tensor.shape()
    assert tt.compression_ratio() > 15.0 and tt.compression_ratio() == 16.0
    ot = O.quantize_ternary(np.array(data, dtype=np.float32).reshape(2, 4))
    assert (tt.packed_data == ot.packed_data).all()
    assert tt.scale == ot.scale and tt.threshold == ot.threshold
    assert same_bits(deq.numpy(), O.dequantize_ternary(ot))


def test_ternary_bit_access(provider):                            # quantization.rs:348-361
    tt = provider.quantizer().quantize_ternary(Tensor.from_data([1.5, -2.0, 0.1, -0.05], [4]))
    assert [tt.get_value(i) for i in range(4)] == [1, -1, 0, 0]
    assert tt.get_value(4) == 0 and tt.memory_size() == 1 and tt.element_count == 4


def test_quantizer_rejects_non_f32(provider):
    with pytest.raises(Error, match="BitNet quantization requires FP32 input tensors"):
        provider.quantizer().quantize_ternary(Tensor.from_data([1, 2, 3, 4], [4], DataType.I8))
    with pytest.raises(Error, match="outside this build"):
        provider.quantizer().quantize_binary(Tensor.from_data([1, 2, 3, 4], [4]))


# ---- allocator.rs tests ---------------------------------------------------------------------------

def test_allocator(provider):                                     # allocator.rs:218-292
    alloc = create_bitnet_provider().get_allocator()
    info = alloc.get_memory_info()
    assert info.allocated_bytes == 0 and info.peak_bytes == 0 and info.total_bytes > 2 ** 37
    buf = alloc.allocate([1000], DataType.Bool)
    assert buf.size == 125 and buf.alignment == 32 and buf.ptr % 32 == 0
    info = alloc.get_memory_info()
    assert info.allocated_bytes == 125 and info.peak_bytes == 125
    alloc.deallocate(buf)
    info = alloc.get_memory_info()
    assert info.allocated_bytes == 0 and info.peak_bytes == 125
    t = alloc.allocate([100], DataType.U8)
    assert t.size == 25 and t.alignment == 32
    alloc.deallocate(t)
    m = alloc.allocate([32, 32], DataType.Bool)
    assert m.size == 128
    alloc.deallocate(m)
    f = alloc.allocate([10, 10], DataType.F16)
    assert f.size == 200 and f.alignment == 16
    alloc.deallocate(f)
    with pytest.raises(Error, match="Unsupported data type for BitNet allocator"):
        alloc.allocate([4], DataType.I32)


def test_execute_with_weights_from_a_packed_file(provider, tmp_path):
    """Ternarise once, save, load, execute: same bits as execute() on the f32 weights."""
    from ronn_amd.bitnet import BitNetQuantizer, TernaryTensor
    a = synth_normal(71, 1.0, (5, 300))
    w = synth_normal(72, 0.02, (300, 77))
    tw = BitNetQuantizer(QuantizationMethod.Ternary, provider).quantize_ternary(Tensor.from_data(w, [300, 77]))
    path = tmp_path / "layer.rbnt"
    tw.save(path)
    loaded = TernaryTensor.load(path)
    assert loaded.shape == [300, 77] and (loaded.packed_data == tw.packed_data).all()
    kernel = provider.create_ternary_matmul_kernel(0, 0, 0)
    want = kernel.execute([Tensor.from_data(a, [5, 300]), Tensor.from_data(w, [300, 77])])[0].numpy()
    got = kernel.execute_prepacked(Tensor.from_data(a, [5, 300]), loaded).numpy()
    assert got.shape == (5, 77) and same_bits(got, want)
    assert kernel.get_performance_stats().execution_count == 2
    with pytest.raises(Error, match="Matrix dimension mismatch"):
        kernel.execute_prepacked(Tensor.from_data(a[:, :299].copy(), [5, 299]), loaded)
