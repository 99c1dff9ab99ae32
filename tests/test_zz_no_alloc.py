"""The entry point that allocates nothing, rbn_gemm_t2_i8_skinny_static, against
rbn_gemm_t2_i8_skinny through the C ABI: same int32 accumulators and same f32 bits, on calls in
a row that share the library's static scratch array (the later ones with smaller inputs, so
they find the earlier ones' partial tiles and counters in it)."""
import numpy as np
import pytest

from ronn_amd import _lib
from ronn_amd.device import synth_normal

pytestmark = pytest.mark.gpu


def operands(ctx, M, K, N, seed):
    x = synth_normal(0x5EED0061 + seed, 1.0, (M, K))
    w = synth_normal(0x5EED1061 + seed, 0.02, (K, N))
    d_p, w_scale, _, _ = ctx.quantize_ternary(ctx.to_device(w), w.size)
    d_t = ctx.tile_weights(d_p, K, N)
    acts = ctx.act_quant_i8(ctx.to_device(x), M, K)
    return acts, d_t, w_scale


def both(ctx, M, K, N, seed):
    acts, d_t, w_scale = operands(ctx, M, K, N, seed)
    want_out, want_acc = ctx.skinny(acts, d_t, w_scale, M, K, N, want_acc=True)
    got_out, got_acc = ctx.skinny_static(acts, d_t, w_scale, M, K, N, want_acc=True)
    ctx.sync()
    n = M * N
    assert (got_acc.download(np.int32, n) == want_acc.download(np.int32, n)).all(), (M, K, N)
    assert (got_out.download(np.uint32, n) == want_out.download(np.uint32, n)).all(), (M, K, N)
    assert np.abs(want_acc.download(np.int32, n)).max() > 0


def test_static_scratch_matches_on_consecutive_calls(ctx):
    # every shape here is narrow enough to be split along k across workgroups, so the partial
    # tiles and the ticket counters really go through the static array (6, 2 and 4 parts);
    # the second and third call are smaller than the first
    for seed, (M, K, N) in enumerate(((16, 11008, 512), (8, 4096, 1024), (40, 8192, 256), (16, 11008, 512))):
        print("static scratch", M, K, N, flush=True)
        both(ctx, M, K, N, seed)
    # a wide matrix is not split and needs no scratch: same entry point, same bits
    both(ctx, 4, 1024, 16384, 9)


def test_static_call_under_graph_capture_allocates_nothing(ctx):
    # captured in a HIP graph (where an allocation would be an error) and replayed three times with
    # eager work in between: every replay gives the eager entry point's bits, and the library's
    # device-memory accounting does not move across capture and replays
    M, K, N = 16, 11008, 512                     # split along k: partial tiles and tickets in the static array
    acts, d_t, w_scale = operands(ctx, M, K, N, 21)
    want_out, want_acc = ctx.skinny(acts, d_t, w_scale, M, K, N, want_acc=True)
    d_out, d_acc = ctx.alloc(4 * M * N), ctx.alloc(4 * M * N)
    ctx.sync()
    before = ctx.memory_info()
    ctx.graph_begin()
    ctx.skinny_static(acts, d_t, w_scale, M, K, N, d_out=d_out, d_acc=d_acc)
    graph = ctx.graph_end()
    assert ctx.memory_info() == before
    n = M * N
    for replay in range(3):
        ctx.lib.rbn_fill_u8(ctx.handle, d_out.ptr, 0xFF, 4 * n)
        ctx.graph_launch(graph)
        ctx.sync()
        assert (d_acc.download(np.int32, n) == want_acc.download(np.int32, n)).all(), replay
        assert (d_out.download(np.uint32, n) == want_out.download(np.uint32, n)).all(), replay
        both(ctx, 8, 4096, 1024, 30 + replay)     # eager work on the same scratch between replays
    assert ctx.memory_info()[0] >= before[0]      # (the eager calls above allocate their own operands)
    ctx.graph_destroy(graph)


def test_static_scratch_belongs_to_one_context_per_gpu(ctx):
    # `ctx` has used the array above; another context on the same GPU is refused until `ctx` goes
    from ronn_amd.device import Context
    both(ctx, 8, 4096, 1024, 40)
    with Context(0) as other:
        d = other.alloc(65536)
        rc = other.lib.rbn_gemm_t2_i8_skinny_static(other.handle, d.ptr, d.ptr, d.ptr, d.ptr, 1.0, 1, 64, 64, None,
                                                    d.ptr)
        assert rc == _lib.RBN_ERR_INVALID
        assert "in use by another context" in other.lib.rbn_last_error().decode()
    both(ctx, 8, 4096, 1024, 41)


def test_static_scratch_refuses_what_does_not_fit(ctx):
    # 127 column groups x 3 parts x 4 row tiles = 1524 partial tiles > 1024: refused on the
    # host, nothing is launched
    M, K, N = 64, 8192, 127 * 64
    d = ctx.alloc(4096)
    rc = ctx.lib.rbn_gemm_t2_i8_skinny_static(ctx.handle, d.ptr, d.ptr, d.ptr, d.ptr, 1.0, M, K, N, None, d.ptr)
    assert rc == _lib.RBN_ERR_UNSUPPORTED
    msg = ctx.lib.rbn_last_error().decode()
    assert "1524 partial tiles" in msg and "1024 tiles" in msg
    with pytest.raises(_lib.RbnError):
        ctx.skinny_static((d, d, d), d, 1.0, 65, 64, 64)
