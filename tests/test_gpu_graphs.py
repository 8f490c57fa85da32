"""The quantized-linear chains under HIP graph capture: every kernel is stream-ordered and allocation-free, so a chain
whose buffers come from the graph's private pool can be captured once and replayed.  Replays are interleaved with eager
work and synchronisations and every replay is compared bit for bit with the eager result (under capture the dynamic FP8
quantiser records its three barrier-free kernels instead of the one-launch kernel with the grid barrier; no memset node is
involved)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(dev):
    from lyradiff_amd import ops as _ops

    return _ops


def test_flux_mlp_fp8_chain_replays_exactly(ops, dev):
    m, d, h = 1024, 3072, 12288
    g = torch.Generator().manual_seed(5)
    w_up, s_up = ops.fp8_quant((torch.randn(h, d, generator=g) * 0.02).bfloat16().to(dev))
    w_dn, s_dn = ops.fp8_quant((torch.randn(d, h, generator=g) * 0.02).bfloat16().to(dev))
    wp_up, wp_dn = ops.repack_weight(w_up), ops.repack_weight(w_dn)
    b_up = (torch.randn(h, generator=g) * 0.02).bfloat16().to(dev)
    b_dn = (torch.randn(d, generator=g) * 0.02).bfloat16().to(dev)
    x = torch.randn(m, d, generator=g).bfloat16().to(dev)

    def chain(inp):
        q, s = ops.fp8_quant(inp)
        hid = ops.fp8_linear(q, wp_up, s, s_up, b_up, True)
        q2, s2 = ops.fp8_quant(hid)
        return ops.fp8_linear(q2, wp_dn, s2, s_dn, b_dn, False)

    side = torch.cuda.Stream()
    static_x = x.clone()
    with torch.cuda.stream(side):
        chain(static_x)  # warm-up on the capture stream
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        static_y = chain(static_x)
    for i in range(4):
        xi = (x * (1.0 + 0.25 * i)).bfloat16()
        eager = chain(xi)
        torch.cuda.synchronize()
        static_x.copy_(xi)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager), f"replay {i} differs from the eager result"
        # unrelated eager work between replays
        ops.sq_quant_dynamic(x.half(), None)
        torch.cuda.synchronize()


@pytest.mark.parametrize("panels", [False, True])
def test_flux_mlp_fp8_running_maximum_chain_replays_exactly(ops, dev, panels):
    """The chain bench.py times -- persistent GEMM that leaves its largest output, GELU + quantisation in one pass that also
    clears the other maximum slot -- captured as two steps (so both slots take both roles) and replayed."""
    m, d, h = 1024, 3072, 12288  # 192 tiles of 256x256: the up projection runs tactic 6/4; the persistent kernel is forced below
    g = torch.Generator().manual_seed(8)
    w_up, s_up = ops.fp8_quant((torch.randn(h, d, generator=g) * 0.02).bfloat16().to(dev))
    w_dn, s_dn = ops.fp8_quant((torch.randn(d, h, generator=g) * 0.02).bfloat16().to(dev))
    wp_up, wp_dn = ops.repack_weight(w_up), ops.repack_weight(w_dn)
    b_up = (torch.randn(h, generator=g) * 0.02).bfloat16().to(dev)
    b_dn = (torch.randn(d, generator=g) * 0.02).bfloat16().to(dev)
    x = torch.randn(m, d, generator=g).bfloat16().to(dev)
    slots = [torch.zeros(1, dtype=torch.float32, device=dev) for _ in range(2)]

    def step(inp, k):
        if panels:  # quantised activations as k-panels, as bench.py passes them
            q, s = ops.fp8_quant_panels(inp)
            with ops.gemm_thread_tactic(7):
                u = ops.fp8_linear_panels(q, wp_up, s, s_up, b_up, slots[k % 2])
            q2, s2 = ops.fp8_gelu_quant_panels(u, slots[k % 2], clear_max=slots[(k + 1) % 2])
            return ops.fp8_linear_panels(q2, wp_dn, s2, s_dn, b_dn)
        q, s = ops.fp8_quant(inp)
        with ops.gemm_thread_tactic(7):
            u = ops.fp8_linear_max(q, wp_up, s, s_up, b_up, slots[k % 2])
        q2, s2 = ops.fp8_gelu_quant(u, slots[k % 2], clear_max=slots[(k + 1) % 2])
        return ops.fp8_linear(q2, wp_dn, s2, s_dn, b_dn, False)

    def two_steps(inp):
        return step(inp, 0), step(inp * 2, 1)

    side = torch.cuda.Stream()
    static_x = x.clone()
    with torch.cuda.stream(side):
        two_steps(static_x)  # warm-up on the capture stream; leaves slot 0 cleared for the next step 0
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        static_y = two_steps(static_x)
    for i in range(3):
        xi = (x * (1.0 + 0.25 * i)).bfloat16()
        eager = two_steps(xi)
        torch.cuda.synchronize()
        static_x.copy_(xi)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y[0], eager[0]) and torch.equal(static_y[1], eager[1]), f"replay {i} differs from the eager result"
        ops.sq_quant_dynamic(x.half(), None)  # unrelated eager work between replays
        torch.cuda.synchronize()


def test_sdxl_int8_ffn_chain_replays_exactly(ops, dev):
    m, d, inner = 4096, 640, 2560
    g = torch.Generator().manual_seed(6)
    w_up = ops.repack_weight(torch.randint(-127, 128, (2 * inner, d), generator=g, dtype=torch.int8).to(dev))
    w_dn = ops.repack_weight(torch.randint(-127, 128, (d, inner), generator=g, dtype=torch.int8).to(dev))
    ws_up = (torch.rand(2 * inner, generator=g) * 9e-4 + 1e-4).to(dev)
    ws_dn = (torch.rand(d, generator=g) * 9e-3 + 1e-3).to(dev)
    gamma = torch.ones(d, dtype=torch.float16, device=dev)
    beta = torch.zeros(d, dtype=torch.float16, device=dev)
    x = torch.randn(m, d, generator=g).half().to(dev)

    def chain(inp):
        q, s, _ = ops.layernorm_int8(inp, gamma, beta, None, None)
        hid = ops.int8_linear(q, w_up, ws_up, s, None, torch.float16)
        q2, s2 = ops.geglu_int8_dynamic(hid, None, None)
        return ops.int8_linear(q2, w_dn, ws_dn, s2, None, torch.float16)

    side = torch.cuda.Stream()
    static_x = x.clone()
    with torch.cuda.stream(side):
        chain(static_x)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        static_y = chain(static_x)
    for i in range(3):
        xi = torch.roll(x, i + 1, 0)
        eager = chain(xi)
        static_x.copy_(xi)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager), f"replay {i} differs from the eager result"
    # replay cost of the launch-bound chain (informative): four kernels without Python between them
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    print(f"SDXL INT8 FFN chain, graph replay: {e0.elapsed_time(e1) / 20 * 1e3:.1f} us per chain")


_FIRST_CALL_UNDER_CAPTURE = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
from lyradiff_amd import ops
from oracle import oracle as O
dev = torch.device("cuda:0")
g = torch.Generator().manual_seed(11)
x = (torch.randn(96, 2 * 640, generator=g) * 2).half().to(dev)
side = torch.cuda.Stream()
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph, stream=side):   # the process's very first GEGLU call: the gate table is not built yet
    q_static, s_static = ops.geglu_int8_dynamic(x, None, None)
for i in range(3):
    graph.replay()
    torch.cuda.synchronize()
    q_ref, s_ref = O.geglu_int8_dynamic(x.float().cpu().numpy(), None, None, "f16")
    assert (q_static.cpu().numpy() == q_ref).all() and (s_static.cpu().numpy() == s_ref).all(), i
    x.copy_(torch.roll(x, 1, 0))
q_eager, s_eager = ops.geglu_int8_dynamic(x, None, None)   # first eager call: builds the table for good
graph.replay()
torch.cuda.synchronize()
assert torch.equal(q_eager, q_static) and torch.equal(s_eager, s_static)
print("capture-first ok")
"""


def test_geglu_first_call_inside_a_capture(dev):
    """The GEGLU gate table is built by the first call on a device.  When that call is being captured into a graph it must
    not block: the table kernel is recorded into the graph instead, and replays are exact.  Needs a process of its own (in
    this one the table exists already)."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", _FIRST_CALL_UNDER_CAPTURE, root], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "capture-first ok" in r.stdout, r.stdout + r.stderr
