"""The entry point that allocates nothing: gguf_mmq_static against gguf_mmq_engine, through the C ABI.

Collected last (the file name sorts behind every other test file), so a failure here hides nothing."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as o
from vllm_gguf_plugin_prism_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu


def _rows_bytes(m, k):
    """Bytes the quantized rows take in the library's own array (see include/gguf_hip.h)."""
    return (m * ((k + 511) // 512 * 512) // 32 * 44 + 255) // 256 * 256


def _both(w, x, qtype, n):
    """(result of gguf_mmq_static, result of gguf_mmq_engine with the same room for partial tiles)."""
    h = _lib.lib()
    m, k = x.shape
    cap = h.gguf_mmq_static_capacity()
    assert cap == 32 << 20
    stream = torch.cuda.current_stream().cuda_stream
    y_static = torch.full((m, n), float("nan"), dtype=x.dtype, device="cuda")
    rc = h.gguf_mmq_static(w.data_ptr(), x.data_ptr(), ops._code(x.dtype), y_static.data_ptr(), qtype, n, k, m, stream)
    assert rc == 0
    rows_public = (m * h.gguf_q8_1_row_bytes(k) + 255) // 256 * 256
    nbytes = rows_public + (cap - _rows_bytes(m, k))          # same number of bytes behind the rows as the static array has
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    y_ref = torch.full((m, n), float("nan"), dtype=x.dtype, device="cuda")
    rc = h.gguf_mmq_engine(w.data_ptr(), x.data_ptr(), ops._code(x.dtype), ws.data_ptr(), y_ref.data_ptr(), qtype, n, k, m,
                           ops.MMQ_ENGINES["auto"], nbytes, stream)
    assert rc == 0
    torch.cuda.synchronize()
    return y_static, y_ref


def test_static_entry_point_matches_on_two_calls_the_second_smaller():
    rng = np.random.default_rng(4242)
    # first call: 56 tiles with a long K, so the plan splits K and the fp32 partial tiles go through the array
    n1, k1, m1 = 1792, 4096, 200
    w1 = torch.from_numpy(o.make_weights(rng, o.Q6_K, n1, k1)).cuda()
    x1 = torch.from_numpy(rng.standard_normal((m1, k1)).astype(np.float32)).cuda()
    a, b = _both(w1, x1, o.Q6_K, n1)
    assert torch.equal(a, b)
    exp = o.mul_mat_a8(w1.cpu().numpy(), x1.cpu().numpy(), o.Q6_K, n1, "mmq")
    assert o.rel_l2(a.cpu().numpy(), exp) <= 1e-5
    # second call, smaller in every dimension, another format and dtype: whatever the first call left in the array
    # must not show
    n2, k2, m2 = 200, 512, 37
    w2 = torch.from_numpy(o.make_weights(rng, o.Q4_K, n2, k2)).cuda()
    x2 = torch.from_numpy(rng.standard_normal((m2, k2)).astype(np.float32)).to(torch.float16).cuda()
    a, b = _both(w2, x2, o.Q4_K, n2)
    assert torch.equal(a, b)
    exp = o.mul_mat_a8(w2.cpu().numpy(), x2.float().cpu().numpy(), o.Q4_K, n2, "mmq")
    assert o.rel_l2(a.float().cpu().numpy(), exp) <= 1e-3
    # a handful of rows takes the streaming kernel inside both entry points
    a, b = _both(w2, x2[:3].contiguous(), o.Q4_K, n2)
    assert torch.equal(a, b)


def test_static_entry_point_rejects_what_does_not_fit():
    h = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    w = torch.zeros(16, dtype=torch.uint8, device="cuda")
    # 4096 rows of K = 18944: 4096 * 19456 / 32 * 44 bytes of quantized rows, more than 32 MiB
    assert h.gguf_mmq_static(w.data_ptr(), w.data_ptr(), 1, w.data_ptr(), o.Q6_K, 64, 18944, 4096, stream) == -6
    assert h.gguf_mmq_static(w.data_ptr(), w.data_ptr(), 1, w.data_ptr(), 99, 64, 256, 4, stream) == -1
    assert h.gguf_mmq_static(w.data_ptr(), w.data_ptr(), 1, w.data_ptr(), o.Q6_K, 64, 100, 4, stream) == -3
    torch.cuda.synchronize()
