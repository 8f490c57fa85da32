"""The allocation-free entry point lq_fp8_amax_cast_static against lq_fp8_amax_cast, through the C ABI: bit-identical
codes and scale, on calls in a row that share the static scratch array (the second smaller than the first), for every
element type, odd sizes and the size limits."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _call(lib, fn, q, s, x, n):
    from lyradiff_amd.ops import _DT, _stream

    rc = getattr(lib, fn)(C.c_void_p(q.data_ptr()), C.c_void_p(s.data_ptr()), C.c_void_p(x.data_ptr()), _DT[x.dtype], n, _stream())
    return rc


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
def test_static_entry_point_matches_the_allocating_one_on_consecutive_calls(dev, dt):
    from lyradiff_amd import lib as L

    lib = L.load()
    g = torch.Generator().manual_seed(2024)
    # first a large call, then smaller ones: the scratch keeps the previous call's partial maxima, and a stale one
    # (the first tensor has the largest values) would show up as a wrong scale in the next call
    sizes = [4608 * 3072, 1024 * 1280 + 5, 32768, 32769, 4096, 40, 1]
    mags = [8.0, 1.0, 0.5, 0.25, 0.125, 0.06, 0.03]
    xs = [(torch.randn(n, generator=g) * mag).to(dt).to(dev) for n, mag in zip(sizes, mags)]
    # outputs allocated before the calls under test: the entry point itself allocates nothing
    q_new = [torch.zeros(n + 16, dtype=torch.uint8, device=dev) for n in sizes]
    s_new = [torch.zeros(1, dtype=torch.float32, device=dev) for _ in sizes]
    q_old = [torch.zeros(n + 16, dtype=torch.uint8, device=dev) for n in sizes]
    s_old = [torch.zeros(1, dtype=torch.float32, device=dev) for _ in sizes]
    torch.cuda.synchronize()
    for i, n in enumerate(sizes):
        assert _call(lib, "lq_fp8_amax_cast_static", q_new[i], s_new[i], xs[i], n) == 0, lib.lq_last_error()
    for i, n in enumerate(sizes):
        assert _call(lib, "lq_fp8_amax_cast", q_old[i], s_old[i], xs[i], n) == 0, lib.lq_last_error()
    torch.cuda.synchronize()
    for i, n in enumerate(sizes):
        assert s_new[i].item() == s_old[i].item(), (i, n)
        assert torch.equal(q_new[i], q_old[i]), (i, n)
        assert int(q_new[i][n:].max()) == 0  # nothing written past the end
        x = xs[i].float().cpu().numpy()
        if n <= 1024 * 1280 + 5:  # and both equal the oracle
            q_ref, s_ref = O.fp8_amax_cast(x)
            assert s_new[i].item() == float(s_ref) and np.array_equal(q_new[i][:n].cpu().numpy(), q_ref)
    assert lib.lq_fp8_amax_cast_status() == 0


def test_static_entry_point_rejects_what_its_scratch_cannot_hold(dev):
    from lyradiff_amd import lib as L

    lib = L.load()
    limit = lib.lq_fp8_amax_cast_static_max_elems()
    assert limit == 8192 * 32768
    x = torch.zeros(64, dtype=torch.bfloat16, device=dev)
    q = torch.zeros(64, dtype=torch.uint8, device=dev)
    s = torch.zeros(1, dtype=torch.float32, device=dev)
    assert _call(lib, "lq_fp8_amax_cast_static", q, s, x, limit + 1) == -2  # LQ_ERR_SHAPE, before anything is launched
    assert b"static scratch" in lib.lq_last_error()
    assert _call(lib, "lq_fp8_amax_cast_static", q, s, x, 0) == -2
    assert _call(lib, "lq_fp8_amax_cast_static", q, s, x[1:], 32) == -1  # misaligned source: LQ_ERR_ARG
    assert lib.lq_fp8_amax_cast_static(None, C.c_void_p(s.data_ptr()), C.c_void_p(x.data_ptr()), 2, 64, None) == -1
    # all-zero input: scale 0, codes NaN-free? 0 * (1/0) = NaN in both entry points -- they must agree
    q2 = torch.zeros(64, dtype=torch.uint8, device=dev)
    s2 = torch.ones(1, dtype=torch.float32, device=dev)
    assert _call(lib, "lq_fp8_amax_cast_static", q, s, x, 64) == 0 and _call(lib, "lq_fp8_amax_cast", q2, s2, x, 64) == 0
    torch.cuda.synchronize()
    assert s.item() == s2.item() == 0.0 and torch.equal(q, q2)


def test_static_entry_point_in_a_graph_replays_exactly(dev):
    """What the entry point is for: captured into a HIP graph (it allocates nothing, waits for nothing and records no
    memset) and replayed, with eager calls of the allocating entry point between the replays; every replay is compared
    with the eager result."""
    from lyradiff_amd import ops

    g = torch.Generator().manual_seed(7)
    n = 1024 * 3072
    static_x = torch.randn(n, generator=g).bfloat16().to(dev)
    q = torch.zeros(n, dtype=torch.uint8, device=dev)
    s = torch.zeros(1, dtype=torch.float32, device=dev)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        ops.fp8_quant_static(static_x, q, s)  # first use on the device outside the capture (looks up the scratch address)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ops.fp8_quant_static(static_x, q, s)
    for i in range(4):
        xi = (torch.randn(n, generator=g) * (0.5 + i)).bfloat16().to(dev)
        q_eager, s_eager = ops.fp8_quant(xi)
        torch.cuda.synchronize()
        static_x.copy_(xi)
        graph.replay()
        torch.cuda.synchronize()
        assert s.item() == s_eager.item() and torch.equal(q, q_eager), f"replay {i}"
        ops.fp8_quant(xi[: 4096 * (i + 1)])  # unrelated eager work between replays
        torch.cuda.synchronize()
    assert not ops.fp8_amax_cast_status()
