"""The torch operator library `_C_gguf`: schemas as the reference defines them (csrc/torch_bindings.cpp:22-53),
dispatch keys, traced shapes (ops.py:116-175) and the module alias; the GPU tests call the operators through
torch.ops and compare with the direct calls."""
import sys
import types

import numpy as np
import pytest
import torch

from oracle import gguf_oracle as o
from vllm_gguf_plugin_prism_amd import _C_gguf, ops, synth

# csrc/torch_bindings.cpp:23-40, whitespace normalised
REFERENCE_SCHEMAS = {
    "ggml_dequantize": "_C_gguf::ggml_dequantize(Tensor W, int type, SymInt m, SymInt n, ScalarType? dtype) -> Tensor",
    "ggml_mul_mat_vec_a8": "_C_gguf::ggml_mul_mat_vec_a8(Tensor W, Tensor X, int type, SymInt row) -> Tensor",
    "ggml_mul_mat_a8": "_C_gguf::ggml_mul_mat_a8(Tensor W, Tensor X, int type, SymInt row) -> Tensor",
    "ggml_moe_a8": "_C_gguf::ggml_moe_a8(Tensor X, Tensor W, Tensor sorted_token_ids, Tensor expert_ids, "
                   "Tensor num_tokens_post_padded, int type, SymInt row, SymInt top_k, SymInt tokens) -> Tensor",
    "ggml_moe_a8_vec": "_C_gguf::ggml_moe_a8_vec(Tensor X, Tensor W, Tensor topk_ids, int top_k, int type, SymInt row, "
                       "SymInt tokens) -> Tensor",
    "ggml_moe_get_block_size": "_C_gguf::ggml_moe_get_block_size(int type) -> int",
}


def test_schemas_match_the_reference():
    for name, want in REFERENCE_SCHEMAS.items():
        assert str(getattr(torch.ops._C_gguf, name).default._schema) == want


def test_both_bindings_define_the_same_library():
    """The compiled binding is the one in use when it has been built; the Python binding (GGUF_TORCH_BINDING=python)
    defines the same schemas and dispatch keys in a fresh interpreter."""
    import subprocess

    assert _C_gguf.NATIVE == _C_gguf.NATIVE_PATH.exists()
    code = (
        "import torch\n"
        "from vllm_gguf_plugin_prism_amd import _C_gguf\n"
        "assert not _C_gguf.NATIVE\n"
        "for n in ('ggml_dequantize', 'ggml_mul_mat_vec_a8', 'ggml_mul_mat_a8', 'ggml_moe_a8', 'ggml_moe_a8_vec', 'ggml_moe_get_block_size'):\n"
        "    print(getattr(torch.ops._C_gguf, n).default._schema)\n"
        "    print(n, torch._C._dispatch_has_kernel_for_dispatch_key('_C_gguf::' + n, 'CUDA'))\n"
    )
    env = dict(__import__("os").environ, GGUF_TORCH_BINDING="python")
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, cwd=str(_C_gguf.NATIVE_PATH.parent.parent))
    assert res.returncode == 0, res.stderr
    lines = res.stdout.strip().splitlines()
    for i, (name, want) in enumerate(REFERENCE_SCHEMAS.items()):
        assert lines[2 * i] == want
        assert lines[2 * i + 1] == f"{name} {name != 'ggml_moe_get_block_size'}"


def test_dispatch_keys():
    for name in REFERENCE_SCHEMAS:
        op = f"_C_gguf::{name}"
        has_cuda = torch._C._dispatch_has_kernel_for_dispatch_key(op, "CUDA")
        assert has_cuda == (name != "ggml_moe_get_block_size")
        assert not torch._C._dispatch_has_kernel_for_dispatch_key(op, "CPU")
    assert torch._C._dispatch_has_kernel_for_dispatch_key("_C_gguf::ggml_moe_get_block_size", "CompositeExplicitAutograd")


def test_cpu_tensors_are_refused():
    with pytest.raises(NotImplementedError):
        torch.ops._C_gguf.ggml_dequantize(torch.zeros(1, 34, dtype=torch.uint8), o.Q8_0, 1, 32, None)


def test_block_size_needs_no_tensor():
    for qt in (o.Q4_0, o.Q8_0, o.Q4_K, o.Q6_K):
        assert torch.ops._C_gguf.ggml_moe_get_block_size(qt) == ops.ggml_moe_get_block_size(qt)


def test_traced_shapes():
    from torch._subclasses.fake_tensor import FakeTensorMode

    _C_gguf.register_fakes()
    _C_gguf.register_fakes()  # a second call is a no-op
    with FakeTensorMode():
        W = torch.empty(64, 144, dtype=torch.uint8)
        X = torch.empty(3, 256, dtype=torch.bfloat16)
        y = torch.ops._C_gguf.ggml_mul_mat_a8(W, X, o.Q4_K, 64)
        assert y.shape == (3, 64) and y.dtype == torch.bfloat16
        y = torch.ops._C_gguf.ggml_mul_mat_vec_a8(W, X, o.Q4_K, 64)
        assert y.shape == (3, 64) and y.dtype == torch.bfloat16
        d = torch.ops._C_gguf.ggml_dequantize(W, o.Q4_K, 64, 256, None)
        assert d.shape == (64, 256) and d.dtype == torch.float16          # the default dtype, ops.py:124
        d = torch.ops._C_gguf.ggml_dequantize(W, o.Q4_K, 32, 512, torch.float32)
        assert d.shape == (32, 512) and d.dtype == torch.float32
        W3 = torch.empty(4, 64, 144, dtype=torch.uint8)
        ids = torch.empty(3, 2, dtype=torch.int32)
        y = torch.ops._C_gguf.ggml_moe_a8_vec(X, W3, ids, 2, o.Q4_K, 64, 3)
        assert y.shape == (6, 64) and y.dtype == torch.bfloat16
        s = torch.empty(64, dtype=torch.int32)
        y = torch.ops._C_gguf.ggml_moe_a8(X, W3, s, s, s, o.Q4_K, 64, 2, 3)
        assert y.shape == (6, 64) and y.dtype == torch.bfloat16


def test_install_as_aliases_the_module():
    pkg = types.ModuleType("fake_plugin_pkg")
    pkg.__path__ = []
    sys.modules["fake_plugin_pkg"] = pkg
    try:
        _C_gguf.install_as("fake_plugin_pkg._C_gguf")
        from fake_plugin_pkg import _C_gguf as alias  # the form the reference's ops.py:44 uses

        assert alias is _C_gguf
    finally:
        sys.modules.pop("fake_plugin_pkg", None)
        sys.modules.pop("fake_plugin_pkg._C_gguf", None)


@pytest.mark.gpu
@pytest.mark.parametrize("qt", [o.Q8_0, o.Q4_K, o.Q6_K, o.IQ4_XS])
def test_gpu_dense_operators_through_torch_ops(qt):
    rng = np.random.default_rng(qt)
    n, k = 96, 512
    w = torch.from_numpy(synth.make_weights(rng, qt, n, k)).cuda()
    for dtype in (None, torch.float32, torch.bfloat16):
        a = torch.ops._C_gguf.ggml_dequantize(w, qt, n, k, dtype)
        assert a.dtype == (dtype or torch.float16) and torch.equal(a, ops.ggml_dequantize(w, qt, n, k, dtype))
    x1 = torch.from_numpy(rng.standard_normal((2, k)).astype(np.float16)).cuda()
    assert torch.equal(torch.ops._C_gguf.ggml_mul_mat_vec_a8(w, x1, qt, n), ops.ggml_mul_mat_vec_a8(w, x1, qt, n))
    want = o.mul_mat_a8(w.cpu().numpy(), x1.cpu().numpy(), qt, n, path="mmvq")
    assert o.rel_l2(torch.ops._C_gguf.ggml_mul_mat_vec_a8(w, x1, qt, n).float().cpu().numpy(), want) <= 1e-3
    if qt != o.IQ4_XS:   # the reference has a8 GEMM tiles for the standard and K formats only (gguf_kernel.cu:236-287)
        x2 = torch.from_numpy(rng.standard_normal((40, k)).astype(np.float16)).cuda()
        assert torch.equal(torch.ops._C_gguf.ggml_mul_mat_a8(w, x2, qt, n), ops.ggml_mul_mat_a8(w, x2, qt, n))


@pytest.mark.gpu
def test_gpu_moe_operators_through_torch_ops():
    rng = np.random.default_rng(5)
    qt, E, n, k, tokens, top_k = o.Q4_0, 4, 64, 256, 70, 2
    w = torch.from_numpy(np.stack([synth.make_weights(rng, qt, n, k) for _ in range(E)])).cuda()
    x = torch.from_numpy(rng.standard_normal((tokens, k)).astype(np.float16)).cuda()
    ids = torch.from_numpy(np.argsort(-rng.standard_normal((tokens, E)), axis=1)[:, :top_k].astype(np.int32)).cuda()
    got = torch.ops._C_gguf.ggml_moe_a8_vec(x, w, ids, top_k, qt, n, tokens)
    assert got.shape == (tokens * top_k, n) and torch.equal(got, ops.ggml_moe_a8_vec(x, w, ids, top_k, qt, n, tokens))
    blk = torch.ops._C_gguf.ggml_moe_get_block_size(qt)
    s, e, npp = ops.moe_align_block_size(ids, blk, E)
    got = torch.ops._C_gguf.ggml_moe_a8(x, w, s, e, npp, qt, n, top_k, tokens)
    assert torch.equal(got, ops.ggml_moe_a8(x, w, s, e, npp, qt, n, top_k, tokens))
    want = o.moe_a8_vec(x.cpu().numpy(), w.cpu().numpy(), ids.cpu().numpy().reshape(-1), top_k, qt, n, tokens)
    assert o.rel_l2(got.float().cpu().numpy(), want) <= 1e-3
