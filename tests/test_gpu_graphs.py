"""GPU: the operators are captured into HIP graphs and replayed (the reference's ops are graph-capturable,
csrc/gguf/gguf_kernel.cu:24-29: caller's stream, no host synchronisation).  Every replay is compared with the eager
result, with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as o

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fn()                       # warm-up on the capture stream: library handles, LDS-size attributes
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn()
    return graph, out


@pytest.mark.parametrize("case", ["mmvq", "mmq_half", "mmq_half_split", "mmq_int8", "mmq_int8_split", "mmq_16_rows", "dequant_gemm",
                                  "moe_vec_grouped", "moe_vec_blocks_of_16", "moe_vec_few_pairs"])
def test_replays_match_eager(case):
    from vllm_gguf_plugin_prism_amd import ops
    rng = np.random.default_rng(abs(hash(case)) % 1000)
    if case.startswith("moe_vec"):
        # 20 / 6 / 0.25 pairs per expert: blocks of 32 slots, of 16, every pair on its own
        e, t, top_k, n, k = {"moe_vec_grouped": (8, 40, 4, 256, 512), "moe_vec_blocks_of_16": (16, 24, 4, 200, 1024),
                             "moe_vec_few_pairs": (32, 2, 4, 200, 1024)}[case]
        w = _dev(np.stack([o.make_weights(rng, o.Q4_0, n, k) for _ in range(e)]))
        ids = _dev(np.stack([rng.choice(e, size=top_k, replace=False) for _ in range(t)]).astype(np.int32))
        xs = [torch.randn(t, k, dtype=torch.float16, device="cuda") for _ in range(3)]
        x = xs[0].clone()
        fn = lambda: ops.ggml_moe_a8_vec(x, w, ids, top_k, o.Q4_0, n, t)
    else:
        qtype, m, n, k = {"mmvq": (o.Q4_K, 1, 512, 1024), "mmq_half": (o.Q6_K, 96, 384, 1024),
                          "mmq_half_split": (o.Q4_K, 200, 250, 4096), "mmq_int8": (o.Q6_K, 96, 384, 1024),
                          "mmq_int8_split": (o.Q4_K, 200, 250, 4096), "mmq_16_rows": (o.Q4_K, 12, 300, 4096),
                          "dequant_gemm": (o.IQ4_XS, 64, 256, 1024)}[case]
        w = _dev(o.make_weights(rng, qtype, n, k))
        xs = [torch.randn(m, k, dtype=torch.float16, device="cuda") for _ in range(3)]
        x = xs[0].clone()
        if case == "mmvq":
            fn = lambda: ops.ggml_mul_mat_vec_a8(w, x, qtype, n)
        elif case == "dequant_gemm":
            fn = lambda: ops.ggml_dequant_gemm(w, x, qtype, n)
        else:
            engine = "half" if case.startswith("mmq_half") else "int8"
            fn = lambda: ops.ggml_mul_mat_a8(w, x, qtype, n, engine=engine)
    graph, out = _capture(fn)
    for xi in xs:
        x.copy_(xi)
        eager = fn().clone()            # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), case


@pytest.mark.parametrize("case", ["split_k", "few_rows"])
def test_entry_point_without_workspace_replays_match_eager(case):
    """gguf_mmq_static is meant for callers under graph capture: gguf_mmq_static_capacity() is called once beforehand
    (it looks up the address of the library's scratch array), after which a captured call must do no set-up of its own.
    One shape whose K is split (fp32 partial tiles and the second launch go through the array) and one that takes the
    streaming kernel for a handful of rows; two replays each with eager work in between, against the eager result and
    against gguf_mmq_engine."""
    from vllm_gguf_plugin_prism_amd import _lib, ops
    h = _lib.lib()
    assert h.gguf_mmq_static_capacity() == 32 << 20           # before any capture
    rng = np.random.default_rng(77)
    qtype, m, n, k = {"split_k": (o.Q6_K, 200, 1792, 4096), "few_rows": (o.Q4_K, 3, 384, 1024)}[case]
    w = _dev(o.make_weights(rng, qtype, n, k))
    xs = [torch.randn(m, k, dtype=torch.float16, device="cuda") for _ in range(3)]
    x = xs[0].clone()
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")

    def fn():
        rc = h.gguf_mmq_static(w.data_ptr(), x.data_ptr(), ops._code(x.dtype), y.data_ptr(), qtype, n, k, m,
                               torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        return y

    graph, out = _capture(fn)
    for xi in xs:
        x.copy_(xi)
        eager = fn().clone()
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), case
        assert o.rel_l2(out.float().cpu().numpy(), ops.ggml_mul_mat_a8(w, x, qtype, n).float().cpu().numpy()) <= 1e-3


def test_two_launch_moe_layer_replays_match_eager():
    """dispatch.fused_moe_gguf at a few tokens (both expert GEMVs, activation, routing weights and top-k sum in two
    launches with a workspace allocated per call) captured and replayed with eager work in between."""
    from vllm_gguf_plugin_prism_amd import dispatch, ops
    rng = np.random.default_rng(91)
    e, hid, inner, t, top_k, qtype = 16, 1024, 512, 3, 4, o.Q4_K
    w13 = _dev(np.stack([o.make_weights(rng, qtype, 2 * inner, hid) for _ in range(e)]))
    w2 = _dev(np.stack([o.make_weights(rng, qtype, hid, inner) for _ in range(e)]))
    assert ops.moe_vec_layer_takes(qtype, qtype, hid, inner, hid, top_k, t, e)
    ids = _dev(np.stack([rng.choice(e, size=top_k, replace=False) for _ in range(t)]).astype(np.int32))
    wts = torch.rand(t, top_k, device="cuda")
    xs = [torch.randn(t, hid, dtype=torch.float16, device="cuda") * 0.05 for _ in range(3)]
    x = xs[0].clone()
    fn = lambda: dispatch.fused_moe_gguf(x, w13, w2, wts, ids, qtype, qtype, "silu")
    graph, out = _capture(fn)
    for xi in xs:
        x.copy_(xi)
        eager = fn().clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


@pytest.mark.parametrize("e,t,qtype2,route", [(16, 70, o.Q4_K, 1), (4, 160, o.Q6_K, 3)])
def test_tile_route_moe_layer_replays_match_eager(e, t, qtype2, route):
    """dispatch.fused_moe_gguf above 64 tokens with few pairs per expert (quantize, routing sort, both expert GEMMs on
    16-slot tiles and the weighted sum, all inside one call with a workspace allocated per call) captured and replayed
    with eager work in between; the routing changes between replays as well.  The second case is the layer in slot
    order on the dense engine (80 pairs per expert, a Q6_K down projection): six launches, its padding slots and the
    inverse of the sort rewritten by every replay."""
    from vllm_gguf_plugin_prism_amd import _lib, dispatch, ops
    rng = np.random.default_rng(92)
    hid, inner, top_k, qtype = 512, 256, 2, o.Q4_K
    w13 = _dev(np.stack([o.make_weights(rng, qtype, 2 * inner, hid) for _ in range(e)]))
    w2 = _dev(np.stack([o.make_weights(rng, qtype2, hid, inner) for _ in range(e)]))
    assert _lib.lib().gguf_moe_mmq_layer_takes(int(qtype), int(qtype2), hid, inner, hid, top_k, t, e) == route
    routes = [_dev(np.stack([rng.choice(e, size=top_k, replace=False) for _ in range(t)]).astype(np.int32)) for _ in range(3)]
    ids = routes[0].clone()
    wts = torch.rand(t, top_k, device="cuda")
    xs = [torch.randn(t, hid, dtype=torch.float16, device="cuda") * 0.05 for _ in range(3)]
    x = xs[0].clone()
    fn = lambda: dispatch.fused_moe_gguf(x, w13, w2, wts, ids, qtype, qtype2, "silu")
    graph, out = _capture(fn)
    for xi, ri in zip(xs, routes):
        x.copy_(xi)
        ids.copy_(ri)
        eager = fn().clone()
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
