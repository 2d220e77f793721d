"""The entry points enqueue on the current stream and never synchronise, so a caller can capture them in a HIP graph
(torch.cuda.CUDAGraph).  Every replay is checked against the eager result, with eager work and synchronisations of
the program between the replays."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rnd(shape, seed, dtype=torch.bfloat16, mul=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * mul).to(dtype)


def _capture_and_replay(cuda, fn, inputs, fresh_inputs):
    """fn(*inputs) -> tensor.  Captures fn on static input buffers, then replays it three times on new input values."""
    static = [t.clone() for t in inputs]
    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    with torch.cuda.stream(side):
        for _ in range(2):  # warm-up outside the capture (library loading, kernel attributes)
            fn(*static)
    torch.cuda.current_stream(cuda).wait_stream(side)
    torch.cuda.synchronize(cuda)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn(*static)
    for step, new in enumerate(fresh_inputs):
        for dst, src in zip(static, new):
            dst.copy_(src)
        graph.replay()
        got = out.clone()
        want = fn(*[t.clone() for t in new])          # eager work between the replays
        torch.cuda.synchronize(cuda)
        assert torch.equal(got, want), f"replay {step} differs from the eager call"


def test_dense_attention_in_a_graph(cuda):
    import mindiesd
    mk = lambda s: tuple(_rnd((1, 4, 700, 128), s + i).to(cuda) for i in range(3))
    _capture_and_replay(cuda, lambda q, k, v: mindiesd.attention_forward(q, k, v, head_first=True), mk(0), [mk(10), mk(20), mk(30)])


def test_fp8_attention_in_a_graph(cuda):
    from mindiesd.layers.quant import fp8_attention_forward
    mk = lambda s: tuple(_rnd((1, 2, 900, 128), s + i).to(cuda) for i in range(3))
    _capture_and_replay(cuda, lambda q, k, v: fp8_attention_forward(q, k, v, layout="BNSD", recipe="amax"), mk(0), [mk(10), mk(20), mk(30)])


def test_mxfp8_gemm_swiglu_in_a_graph(cuda):
    from mindiesd.layers.quant import mx_quantize, mxfp8_gemm_swiglu
    wq, ws = mx_quantize(_rnd((2 * 264, 512), 5, mul=0.05).to(cuda))
    mk = lambda s: (_rnd((300, 512), s).to(cuda),)
    _capture_and_replay(cuda, lambda x: mxfp8_gemm_swiglu(x, wq, ws), mk(0), [mk(10), mk(20), mk(30)])


def test_block_sparse_attention_in_a_graph(cuda):
    from mindiesd.layers.flash_attn import rainfusion as rf
    s, n = 1100, 2
    nb = (s + 127) // 128
    g = torch.Generator().manual_seed(3)
    mask = (torch.rand(1, n, nb, nb, generator=g) < 0.4).to(torch.int8).to(cuda)
    mk = lambda sd: tuple(_rnd((1, n, s, 128), sd + i).to(cuda) for i in range(3))
    _capture_and_replay(cuda, lambda q, k, v: rf.block_sparse_attention_mask(q, k, v, mask, 128 ** -0.5, "BNSD"),
                        mk(0), [mk(10), mk(20), mk(30)])


def test_first_rainfusion_call_of_a_grid_in_a_graph(cuda):
    """The whole rf_v3 call (permute + pool, mask, pairing, attention through the token table) captured for a latent
    grid that no earlier call has seen: the token table is then built inside the graph, without a host wait."""
    from mindiesd.layers.flash_attn import rainfusion as rf
    warm_grid, grid = (2, 16, 24), (3, 19, 17)      # the second one is used nowhere else in the tests
    n = 2
    mk = lambda g, sd: tuple(_rnd((1, n, g[0] * g[1] * g[2], 128), sd + i).to(cuda) for i in range(3))
    run = lambda g: (lambda q, k, v: rf.bsa_sparse_attention_v3(q, k, v, latent_shape_q=g, sparsity=0.5,
                                                                input_layout="BNSD")[0])
    run(warm_grid)(*mk(warm_grid, 0))               # library load and kernel attributes, on another grid
    torch.cuda.synchronize(cuda)
    assert not any(key[:3] == grid for key in rf._token_order_cache)
    static = [t.clone() for t in mk(grid, 1)]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = run(grid)(*static)
    for step, new in enumerate([mk(grid, 10), mk(grid, 20), mk(grid, 30)]):
        for dst, src in zip(static, new):
            dst.copy_(src)
        graph.replay()
        got = out.clone()
        want = run(grid)(*[t.clone() for t in new])  # eager: builds and caches its own table
        torch.cuda.synchronize(cuda)
        assert torch.equal(got, want), f"replay {step} differs from the eager call"


def test_token_order_is_shared_between_streams_without_a_host_wait(cuda):
    from mindiesd.layers.flash_attn import rainfusion as rf
    grid = (2, 11, 13)
    a = rf.token_order(grid, 5, cuda)
    side = torch.cuda.Stream(device=cuda)
    with torch.cuda.stream(side):
        b = rf.token_order(grid, 5, cuda)           # same table, ordered after its fill by an event
        on_side = b.clone()
    side.synchronize()
    torch.cuda.synchronize(cuda)
    assert a.data_ptr() == b.data_ptr() and torch.equal(on_side, a)
    assert sorted(a.cpu().tolist()) == list(range(2 * 11 * 13 + 5))


def test_two_streams_and_two_threads(cuda):
    """Launches from two host threads on two streams at once (no shared state in the library): each result equals the
    one computed alone."""
    import threading
    import mindiesd
    from mindiesd.layers.flash_attn import rainfusion as rf
    s, n = 900, 2
    nb = (s + 127) // 128
    g = torch.Generator().manual_seed(4)
    mask = (torch.rand(1, n, nb, nb, generator=g) < 0.5).to(torch.int8).to(cuda)
    inputs = [tuple(_rnd((1, n, s, 128), 40 * t + i).to(cuda) for i in range(3)) for t in range(2)]
    alone = [(mindiesd.attention_forward(*x, head_first=True), rf.block_sparse_attention_mask(*x, mask, 128 ** -0.5, "BNSD"))
             for x in inputs]
    torch.cuda.synchronize(cuda)
    results, errors = [None, None], []

    def work(t):
        try:
            st = torch.cuda.Stream(device=cuda)
            with torch.cuda.stream(st):
                outs = []
                for _ in range(8):
                    outs = (mindiesd.attention_forward(*inputs[t], head_first=True),
                            rf.block_sparse_attention_mask(*inputs[t], mask, 128 ** -0.5, "BNSD"))
                st.synchronize()
            results[t] = outs
        except Exception as e:  # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for t in range(2):
        assert torch.equal(results[t][0], alone[t][0]) and torch.equal(results[t][1], alone[t][1])
