"""mindiesd_fp8_v_quant_static (the entry point that allocates nothing: per-channel maxima in a device array inside
the library) against mindiesd_fp8_v_quant (caller-provided workspace), both called through the C ABI.

Two calls in a row on one GPU, the second with a smaller input: the array keeps the first call's contents, so the
second call only gives the right scales if the entry point clears what it uses.  Codes and scales must be identical
bit for bit (the two entry points run the same kernels)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _v(shape, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g)
    x = torch.where(torch.rand(shape, generator=g) < 0.01, x * 8, x)
    return x.to(dtype)


def _both(lib, v, native):
    """-> ((v8t, scale) of the workspace entry point, (v8t, scale) of the static one) for v [B, N, S, 128]."""
    b, n, s, d = v.shape
    s128 = (s + 127) // 128 * 128
    stream = native.stream_ptr(v.device)
    res = []
    for static in (False, True):
        v8t = torch.full((b, n, d, s128), 0xAA, dtype=torch.uint8, device=v.device)
        scale = torch.full((b, n, d), -1.0, dtype=torch.float32, device=v.device)
        args = (v.data_ptr(), v8t.data_ptr(), scale.data_ptr(), native.DTYPE_CODE[v.dtype], b, n, s, d,
                v.stride(0), v.stride(1), v.stride(2))
        if static:
            rc = lib.mindiesd_fp8_v_quant_static(*args, stream)
        else:
            ws = torch.empty(lib.mindiesd_fp8_v_quant_workspace_size(b, n), dtype=torch.uint8, device=v.device)
            rc = lib.mindiesd_fp8_v_quant(*args, ws.data_ptr(), ws.numel(), stream)
        assert rc == 0, (static, rc)
        res.append((v8t, scale))
    torch.cuda.synchronize(v.device)
    return res


def test_static_scratch_matches_workspace_entry_point(cuda):
    from mindiesd import _native
    lib = _native.lib()
    assert lib.mindiesd_fp8_v_quant_static_max_heads() == 4096
    # first call: large values in every channel of 6 (batch, head) pairs; second call: fewer heads, a shorter
    # sequence and values 100 times smaller - maxima left over from the first call would give wrong scales
    big = (_v((2, 3, 1500, 128), 1, torch.bfloat16) * 50).to(cuda)
    small = (_v((1, 2, 333, 128), 2, torch.bfloat16) * 0.5).to(cuda)
    for v in (big, small):
        (want8, want_s), (got8, got_s) = _both(lib, v, _native)
        assert torch.equal(got_s, want_s)
        assert torch.equal(got8, want8)
        amax = v.float().abs().amax(dim=2)
        torch.testing.assert_close(got_s, amax / 448.0, rtol=1e-6, atol=0)  # sanity: the scales are amax/448
    # fp16 and a strided (BSND) view
    v = _v((1, 700, 4, 128), 3, torch.float16).to(cuda).transpose(1, 2)
    (want8, want_s), (got8, got_s) = _both(lib, v, _native)
    assert torch.equal(got_s, want_s) and torch.equal(got8, want8)


def test_static_entry_point_under_graph_capture_allocates_nothing(cuda):
    """The callers the entry point is for: a call recorded into a HIP graph (after one eager call, which resolves the
    array's address), replayed on new values with eager calls of the workspace entry point in between; the
    allocator's byte count does not move across a call."""
    from mindiesd import _native
    lib = _native.lib()
    b, n, s, d = 1, 3, 700, 128
    s128 = (s + 127) // 128 * 128
    v = _v((b, n, s, d), 5, torch.bfloat16).to(cuda)
    v8t = torch.zeros((b, n, d, s128), dtype=torch.uint8, device=cuda)
    scale = torch.zeros((b, n, d), dtype=torch.float32, device=cuda)

    def call():
        return lib.mindiesd_fp8_v_quant_static(v.data_ptr(), v8t.data_ptr(), scale.data_ptr(),
                                               _native.DTYPE_CODE[v.dtype], b, n, s, d, v.stride(0), v.stride(1),
                                               v.stride(2), _native.stream_ptr(cuda))

    assert call() == 0                                # first call on the device: symbol lookup
    torch.cuda.synchronize(cuda)
    before = torch.cuda.memory_allocated(cuda), torch.cuda.memory_reserved(cuda)
    assert call() == 0
    torch.cuda.synchronize(cuda)
    assert (torch.cuda.memory_allocated(cuda), torch.cuda.memory_reserved(cuda)) == before
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert call() == 0
    for seed in (6, 7, 8):
        new = (_v((b, n, s, d), seed, torch.bfloat16) * (seed - 5.5)).to(cuda)
        v.copy_(new)
        graph.replay()
        got8, got_s = v8t.clone(), scale.clone()
        (want8, want_s), _ = _both(lib, new, _native)  # eager work between the replays
        assert torch.equal(got_s, want_s) and torch.equal(got8, want8), f"replay with seed {seed}"


def test_static_scratch_limits_and_errors(cuda):
    from mindiesd import _native
    lib = _native.lib()
    v = torch.zeros((1, 1, 128, 128), dtype=torch.bfloat16, device=cuda)
    v8t = torch.empty((1, 1, 128, 128), dtype=torch.uint8, device=cuda)
    sc = torch.empty((1, 1, 128), dtype=torch.float32, device=cuda)
    stream = _native.stream_ptr(v.device)
    # more (batch, head) pairs than the array holds: refused before anything is launched
    rc = lib.mindiesd_fp8_v_quant_static(v.data_ptr(), v8t.data_ptr(), sc.data_ptr(), 0, 4097, 1, 128, 128, 0, 0, 128, stream)
    assert rc == 3
    rc = lib.mindiesd_fp8_v_quant_static(v.data_ptr(), v8t.data_ptr(), sc.data_ptr(), 0, 1, 1, 128, 64, 0, 0, 128, stream)
    assert rc == 2
    rc = lib.mindiesd_fp8_v_quant_static(None, v8t.data_ptr(), sc.data_ptr(), 0, 1, 1, 128, 128, 0, 0, 128, stream)
    assert rc == 1
    torch.cuda.synchronize(cuda)
