"""GPU test of the entry point that allocates nothing: catcoc_launch_quant_matmul_reduce_scatter_static_scratch
against catcoc_launch_quant_matmul_reduce_scatter with a caller-allocated workspace, through the C ABI, bit for bit,
on calls in a row that share the library's built-in scratch (the later ones with smaller inputs)."""
import ctypes as C

import numpy as np
import pytest
import torch

from mm_rs_with_catlass_amd import lib as L
from mm_rs_with_catlass_amd import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(g, M, K, N, P, kr):
    x1 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
    x2 = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=DEV, generator=g)
    s1 = torch.empty(M, device=DEV).uniform_(0.005, 0.02, generator=g)
    s2 = torch.empty(N, device=DEV).uniform_(0.001, 0.01, generator=g)
    bias = torch.randint(-1000, 1000, (N,), dtype=torch.int32, device=DEV, generator=g)
    peers = [torch.randn((kr, N), device=DEV, generator=g) for _ in range(P - 1)]
    return x1, x2, s1, s2, bias, peers


def _both(so, x1, x2, s1, s2, bias, peers, t, d_ws, d_static):
    """-> (out of the existing entry point with its own workspace, out of the static-scratch entry point)."""
    rows = d_ws.keptRows if d_ws.keptRows else t.m // d_ws.rankSize
    outs = []
    for fn, d in ((so.catcoc_launch_quant_matmul_reduce_scatter, d_ws),
                  (so.catcoc_launch_quant_matmul_reduce_scatter_static_scratch, d_static)):
        out = torch.full((rows, t.n), float("nan"), dtype=torch.bfloat16, device=DEV)
        fn(torch.cuda.current_stream().cuda_stream, 0, x1.data_ptr(), x2.data_ptr(), s1.data_ptr(), s2.data_ptr(),
           bias.data_ptr(), None, out.data_ptr(), C.addressof(d), C.byref(t), 0, 0, L.BF16)
        L.check()
        torch.cuda.synchronize()
        outs.append(out)
    return outs


def test_static_scratch_entry_point_matches_the_allocating_one():
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    so = L.load()
    g = torch.Generator(device=DEV).manual_seed(9)
    # (M, K, N, P, kept rows or None = the reduce-scatter path with k-sliced large tiles); later cases are smaller
    cases = [(64, 4096, 2048, 8, 8),        # skinny-M split-K: 16 tiles of 128x128, k slices meet through the scratch
             (16, 2048, 1024, 4, 4),        # smaller, same path: counters and partials where the first call left data
             (1024, 4096, 1024, 4, None),   # k-sliced 128x256 tiles (32 tiles x 8 slices)
             (1024, 2048, 512, 4, None)]    # smaller again
    for M, K, N, P, kr in cases:
        t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
        rows = kr if kr is not None else M // P
        x1, x2, s1, s2, bias, peers = _inputs(g, M, K, N, P, rows)
        mk = lambda: L.make_desc(1 if kr is None else 0, P, [p.data_ptr() for p in peers], N, 0)
        d_ws, d_static = mk(), mk()
        if kr is not None:
            d_ws.keptRows = d_static.keptRows = kr
            need, f, _ = ops.splitk_plan(M, K, N, P, 0, kr)
        else:
            need, f = ops.kslice_plan(L.QUANT_MATMUL_REDUCE_SCATTER, torch.int8, M, K, N, 1, P)
        assert f > 1 and 0 < need <= L.STATIC_SCRATCH_BYTES, "the case must use the scratch"
        ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
        d_ws.workspace, d_ws.workspaceBytes = ws.data_ptr(), need
        d_static.workspace, d_static.workspaceBytes = 0, 0       # ignored by the static-scratch entry point anyway
        want, got = _both(so, x1, x2, s1, s2, bias, peers, t, d_ws, d_static)
        assert not torch.isnan(want.float()).any()
        assert torch.equal(want.view(torch.int16), got.view(torch.int16)), (M, K, N, P, kr)
        if kr is not None:       # the skinny cases are small enough for the CPU oracle: bit for bit against it as well
            import oracle
            _, out_want = oracle.quant_matmul_reduce_scatter(
                x1.cpu().numpy(), x2.cpu().numpy(), s1.cpu().numpy(), s2.cpu().numpy(), bias.cpu().numpy(), 0, kr,
                [p.cpu().numpy() for p in peers], oracle.BF16, want_acc=False)
            assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), out_want), (M, K, N, P, kr)


def test_static_scratch_entry_point_replays_from_a_hip_graph():
    # the callers it is for include code under HIP graph capture: the call records nothing but its kernel (no clearing of
    # the scratch: the counters are zero at load and every launch leaves them at zero), so every replay equals the eager result
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    so = L.load()
    g = torch.Generator(device=DEV).manual_seed(11)
    M, K, N, P, kr = 48, 4096, 1024, 8, 6
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    x1, x2, s1, s2, bias, peers = _inputs(g, M, K, N, P, kr)
    d = L.make_desc(0, P, [p.data_ptr() for p in peers], N, 0)
    d.keptRows = kr
    need, f, _ = ops.splitk_plan(M, K, N, P, 0, kr)
    assert f > 1 and need <= L.STATIC_SCRATCH_BYTES
    out = torch.zeros((kr, N), dtype=torch.bfloat16, device=DEV)

    def call():
        so.catcoc_launch_quant_matmul_reduce_scatter_static_scratch(
            torch.cuda.current_stream().cuda_stream, 0, x1.data_ptr(), x2.data_ptr(), s1.data_ptr(), s2.data_ptr(), bias.data_ptr(),
            None, out.data_ptr(), C.addressof(d), C.byref(t), 0, 0, L.BF16)
    call()
    L.check()
    torch.cuda.synchronize()
    want = out.clone()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        call()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            out.zero_()
            call()
    L.check()
    for _ in range(3):
        out.fill_(1.0)
        call()                                   # eager work between the replays, through the same scratch
        torch.cuda.synchronize()
        out.fill_(2.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_static_scratch_entry_point_rejects_oversized_launches_and_allocates_nothing():
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    so = L.load()
    # 64 x 16 tiles of 128x128 with K > 8192 forces two k slices: 2 * 2048 * 64 KiB of partials > 32 MiB
    M, K, N, P = 2048, 8192 + 256, 8192, 2
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    d = L.make_desc(0, P, [16], N, 0)
    d.keptRows = 8
    so.catcoc_launch_quant_matmul_reduce_scatter_static_scratch(None, 0, 16, 16, 16, 16, None, None, 16, C.addressof(d),
                                                                C.byref(t), 0, 0, L.BF16)
    assert so.catcoc_last_status() != 0 and "built-in scratch holds" in L.last_error()
    # a call that fits allocates nothing: the allocator's statistics do not move and the driver's free memory stays
    g = torch.Generator(device=DEV).manual_seed(10)
    M, K, N, P, kr = 32, 2048, 1024, 8, 4
    t = ops.default_tiling(M, K, N, P, m0=0, n0=0, k0=0)
    x1, x2, s1, s2, bias, peers = _inputs(g, M, K, N, P, kr)
    d = L.make_desc(0, P, [p.data_ptr() for p in peers], N, 0)
    d.keptRows = kr
    out = torch.empty((kr, N), dtype=torch.bfloat16, device=DEV)
    call = lambda: so.catcoc_launch_quant_matmul_reduce_scatter_static_scratch(
        torch.cuda.current_stream().cuda_stream, 0, x1.data_ptr(), x2.data_ptr(), s1.data_ptr(), s2.data_ptr(), bias.data_ptr(),
        None, out.data_ptr(), C.addressof(d), C.byref(t), 0, 0, L.BF16)
    call()
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        call()
    torch.cuda.synchronize()
    L.check()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0
