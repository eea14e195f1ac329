"""GPU parity: q8_1 quantizer, dequantize and MMVQ against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as o

pytestmark = pytest.mark.gpu

SIX = [o.Q4_0, o.Q8_0, o.Q4_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS]
ALL = [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ2_XXS, o.IQ2_XS, o.IQ3_XXS,
       o.IQ1_S, o.IQ4_NL, o.IQ3_S, o.IQ2_S, o.IQ4_XS, o.IQ1_M]
TORCH_DT = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}


def _ops():
    from vllm_gguf_plugin_prism_amd import ops
    return ops


def _to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _x(rng, m, k, dt):
    x32 = rng.standard_normal((m, k)).astype(np.float32)
    t = torch.from_numpy(x32).to(TORCH_DT[dt])
    return t.cuda(), t.to(torch.float32).numpy()  # device tensor, and its exact values as fp32


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("shape", [(1, 1024), (3, 736), (5, 4096), (2, 14336), (70, 256)])
def test_q8_1_bit_exact(shape, dt):
    ops = _ops()
    rng = np.random.default_rng(hash((shape, dt)) % 2**32)
    xd, xv = _x(rng, *shape, dt)
    if shape[0] >= 3:
        xv[1, :64] = 0
        xv[2, 5] = 3.0e4
        xd = torch.from_numpy(xv).to(TORCH_DT[dt]).cuda()
        xv = xd.cpu().to(torch.float32).numpy()
    q, ds = ops.quantize_q8_1(xd)
    qo, do, so = o.quantize_q8_1(xv)
    assert np.array_equal(q.cpu().numpy(), qo)
    assert np.array_equal(ds[:, :, 0].cpu().numpy(), do.astype(np.float32))
    assert np.array_equal(ds[:, :, 1].cpu().numpy(), so.astype(np.float32))


def test_q8_1_ties_round_away_from_zero():
    ops = _ops()
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, :7] = [127.0, 0.5, -0.5, 2.5, -2.5, 1.4990234, np.float32(0.49999997)]
    q, ds = ops.quantize_q8_1(torch.from_numpy(x).cuda())
    assert ds[0, 0, 0].item() == 1.0
    assert q[0, :7].cpu().tolist() == [127, 1, -1, 3, -3, 1, 0]


def test_q8_1_near_ties_and_extreme_scales_bit_exact():
    # Blocks built to sit on the rounding boundary: the block maximum is 127 * d for an arbitrary d, so the scale is d
    # (or its neighbour), and the other values are (k + 1/2) * d and their neighbours one and two units in the last
    # place away.  Scales run from the smallest subnormal quotient to near overflow.
    ops = _ops()
    rng = np.random.default_rng(4242)
    rows = []
    for d in np.concatenate([rng.uniform(0.001, 10.0, 200), 2.0 ** rng.integers(-140, 100, 60), [1.0, 2.0 ** -133, 1e-39, 3e-41, 2.5e36]]).astype(np.float32):
        blk = np.zeros(32, dtype=np.float32)
        k = rng.integers(-126, 126, 31).astype(np.float32)
        base = (k + np.float32(0.5)) * np.float32(d)
        step = rng.integers(-2, 3, 31)
        vals = base.copy()
        for s in (1, 2):
            up = np.nextafter(vals, np.float32(np.inf), dtype=np.float32)
            dn = np.nextafter(vals, np.float32(-np.inf), dtype=np.float32)
            vals = np.where(step >= s, up, np.where(step <= -s, dn, vals))
        blk[:31] = vals
        blk[31] = np.float32(127.0) * np.float32(d)
        rows.append(rng.permutation(blk))
    x = np.stack(rows).astype(np.float32)
    x = x[np.isfinite(x).all(axis=1)]
    x = np.concatenate([x, x[:, ::-1]], axis=1)          # two blocks per row
    q, ds = ops.quantize_q8_1(torch.from_numpy(x).cuda())
    qo, do, so = o.quantize_q8_1(x)
    assert np.array_equal(q.cpu().numpy(), qo)
    assert np.array_equal(ds[:, :, 0].cpu().numpy(), do.astype(np.float32))
    # the same values through the GEMV's own quantizer: Q8_0 weights that pick out one element each
    n, kk = 64, 64
    w = o.make_weights(rng, o.Q8_0, n, kk)
    for r in (0, 17, x.shape[0] - 1):
        xr = torch.from_numpy(x[r : r + 1].copy()).cuda()
        if not np.isfinite(x[r]).all() or np.abs(x[r]).max() > 1e30 or np.abs(x[r]).max() < 1e-30:
            continue
        y = ops.ggml_mul_mat_vec_a8(_to_dev(w), xr, o.Q8_0, n).cpu().numpy()
        exp = o.mul_mat_a8(w, x[r : r + 1], o.Q8_0, n, "mmvq")
        assert o.rel_l2(y, exp) <= 1e-5


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("qtype", ALL)
def test_dequantize_bit_exact(qtype, dt):
    ops = _ops()
    rng = np.random.default_rng(100 + qtype)
    for n, k, raw in [(16, 1024, False), (8, 256, True), (3, 2304, True)]:
        w = o.random_blocks(rng, qtype, n, k) if raw else o.make_weights(rng, qtype, n, k)
        out = ops.ggml_dequantize(_to_dev(w), qtype, n, k, TORCH_DT[dt])
        exp = o.dequantize(w, qtype, dt, "ref")
        if dt == "bf16":
            got = out.view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1)
        else:
            got = out.cpu().numpy().reshape(-1)
        assert got.dtype == exp.dtype
        assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), (o.TYPE_NAMES[qtype], dt, n, k)


def test_dequantize_default_dtype_and_shape_label():
    ops = _ops()
    rng = np.random.default_rng(7)
    w = o.make_weights(rng, o.Q8_0, 6, 64)
    out = ops.ggml_dequantize(_to_dev(w), o.Q8_0, 64, 6, None)  # (m, n) only label m*n outputs
    assert out.dtype == torch.float16 and out.shape == (64, 6)
    assert np.array_equal(out.cpu().numpy().reshape(-1), o.dequantize(w, o.Q8_0, "f16"))


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("m", [1, 2, 3, 5, 8, 9, 10, 11, 16])   # past eight rows: passes of eight, then 1, 2, 3 rows or none
def test_mmvq_matches_a8_oracle(qtype, m):
    ops = _ops()
    rng = np.random.default_rng(200 + qtype * 16 + m)
    for n, k in [(64, 1024), (37, 768), (130, 4096)]:
        if k % o.QUANT_SIZES[qtype][0]:
            continue
        w = o.make_weights(rng, qtype, n, k)
        xd, xv = _x(rng, m, k, "f32")
        y = ops.ggml_mul_mat_vec_a8(_to_dev(w), xd, qtype, n)
        assert y.shape == (m, n) and y.dtype == torch.float32
        exp = o.mul_mat_a8(w, xv, qtype, n, "mmvq")
        err = o.rel_l2(y.cpu().numpy(), exp)
        assert err <= 1e-5, (o.TYPE_NAMES[qtype], m, n, k, err)   # fp32 output: only summation order differs


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("qtype", ALL)
def test_mmvq_half_outputs_within_tolerance(qtype, dt):
    # stated tolerance: rel-L2 <= 1e-3 for fp16 outputs (bf16: 4e-3, its rounding alone is 2^-9) vs the a8 oracle
    ops = _ops()
    rng = np.random.default_rng(300 + qtype)
    n, k, m = 256, 2048, 4
    w = o.make_weights(rng, qtype, n, k)
    xd, xv = _x(rng, m, k, dt)
    y = ops.ggml_mul_mat_vec_a8(_to_dev(w), xd, qtype, n).to(torch.float32).cpu().numpy()
    exp = o.mul_mat_a8(w, xv, qtype, n, "mmvq")
    assert o.rel_l2(y, exp) <= (1e-3 if dt == "f16" else 4e-3)
    # vs unquantized activations the gap is the q8_1 noise itself (~5e-3); the reference gates it with
    # atol=1, rtol=1e-1 on O(1) outputs, scaled here to the output magnitude of the synthetic weights
    full = o.mul_mat_f32(w, xv, qtype, n)
    assert o.rel_l2(y, full) <= 2e-2
    assert np.all(np.abs(y - full) <= np.abs(full).mean() + 1e-1 * np.abs(full))


def test_config1_q8_0_qwen_mlp_shape():
    # BASELINE config 1: Q8_0 [3072,1024], x fp16 [1,1024]
    ops = _ops()
    rng = np.random.default_rng(0)
    w = o.make_weights(rng, o.Q8_0, 3072, 1024)
    wd = _to_dev(w)
    deq = ops.ggml_dequantize(wd, o.Q8_0, 3072, 1024, torch.float16)
    assert np.array_equal(deq.cpu().numpy().reshape(-1), o.dequantize(w, o.Q8_0, "f16"))
    xd, xv = _x(rng, 1, 1024, "f16")
    y = ops.ggml_mul_mat_vec_a8(wd, xd, o.Q8_0, 3072).to(torch.float32).cpu().numpy()
    assert o.rel_l2(y, o.mul_mat_a8(w, xv, o.Q8_0, 3072)) <= 1e-3
    assert o.rel_l2(y, o.mul_mat_f32(w, xv, o.Q8_0, 3072)) <= 2e-2


@pytest.mark.parametrize("shape", [(4096, 4096), (14336, 4096), (4096, 14336)])
def test_config2_q4_k_full_size(shape):
    # full-size Llama-3-8B projections; the oracle on all rows costs seconds in BLAS
    ops = _ops()
    n, k = shape
    rng = np.random.default_rng(1)
    w = o.make_weights(rng, o.Q4_K, n, k)
    wd = _to_dev(w)
    for m in (1, 2):
        xd, xv = _x(rng, m, k, "f16")
        y = ops.ggml_mul_mat_vec_a8(wd, xd, o.Q4_K, n).to(torch.float32).cpu().numpy()
        assert o.rel_l2(y, o.mul_mat_a8(w, xv, o.Q4_K, n, "mmvq")) <= 1e-3
    # linearity in x holds exactly for the dequantized-weight product; with q8_1 it holds to quantization noise
    xa, va = _x(rng, 1, k, "f16")
    y1 = ops.ggml_mul_mat_vec_a8(wd, xa, o.Q4_K, n).float()
    y2 = ops.ggml_mul_mat_vec_a8(wd, (xa * 2).to(torch.float16), o.Q4_K, n).float()
    assert o.rel_l2(y2.cpu().numpy(), 2 * y1.cpu().numpy()) <= 2e-3


@pytest.mark.parametrize("shape", [(4096, 4096), (14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [4, 8])
def test_config2_q4_k_full_size_batch_4_and_8(shape, m):
    """The batch sweep of config 2 at its real shapes through the reference's dispatch policy (linear.py:38-49): batch 4
    on the 4096-row matrices is a GEMV, everything else here goes to ggml_mul_mat_a8, whose offset term uses the stored
    block sums.  The oracle follows the path the policy names."""
    from vllm_gguf_plugin_prism_amd import dispatch as D
    n, k = shape
    rng = np.random.default_rng(21 + m)
    w = o.make_weights(rng, o.Q4_K, n, k)
    xd, xv = _x(rng, m, k, "f16")
    path = D.select_mul_mat_path(o.Q4_K, m, n)
    assert path == ("mmvq" if (n <= 5120 and m <= 6) else "mmq")
    y = D.fused_mul_mat_gguf(xd, _to_dev(w), o.Q4_K)
    assert y.shape == (m, n) and y.dtype == torch.float16
    assert o.rel_l2(y.float().cpu().numpy(), o.mul_mat_a8(w, xv, o.Q4_K, n, path)) <= 1e-3


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K, o.Q6_K, o.Q4_0, o.Q8_0])
def test_mmvq_five_rows_or_more_of_a_large_matrix(qtype, dt):
    """From five rows on (nine for Q4_0 / Q8_0), a matrix of at least 8M weights runs the GEMV operator on 16-row MFMA
    tiles read from the packed blocks (16 rows per launch), with the GEMV's arithmetic: for Q4_K / Q5_K the offset term multiplies
    d8 * sum(q8), not the stored block sum of the tile operator (the two differ by about 1e-2 on these weights).  A
    matrix below that size and K beyond 4096 (no room for partial tiles in this operator's workspace) stay on the
    streaming kernel; all must agree with the GEMV oracle."""
    ops = _ops()
    rng = np.random.default_rng(1600 + qtype)
    tol = 1e-5 if dt == "f32" else 1e-3
    for n, k, ms in [(2048, 4096, (5, 16, 21, 40)), (1100, 8192, (6,)), (300, 1024, (7,))]:
        w = o.make_weights(rng, qtype, n, k)
        wd = _to_dev(w)
        for m in ms:
            xd, xv = _x(rng, m, k, dt)
            y = ops.ggml_mul_mat_vec_a8(wd, xd, qtype, n)
            want = o.mul_mat_a8(w, xv, qtype, n, "mmvq")
            assert o.rel_l2(y.float().cpu().numpy(), want) <= tol, (o.TYPE_NAMES[qtype], n, k, m)
    # with bias, into a column slice of a wider result
    n, k, m = 2048, 4096, 9
    w = o.make_weights(rng, qtype, n, k)
    xd, xv = _x(rng, m, k, dt)
    bias = torch.from_numpy(rng.standard_normal(n).astype(np.float32)).to(TORCH_DT[dt]).cuda()
    wide = torch.full((m, n + 8), 3.0, dtype=TORCH_DT[dt], device="cuda")
    ops.ggml_mul_mat_vec_a8(_to_dev(w), xd, qtype, n, out=wide[:, 8:], bias=bias)
    want = o.mul_mat_a8(w, xv, qtype, n, "mmvq") + bias.float().cpu().numpy()
    assert o.rel_l2(wide[:, 8:].float().cpu().numpy(), want) <= tol
    assert torch.all(wide[:, :8] == 3.0)


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K])
@pytest.mark.parametrize("kind", ["offset", "positive", "negative"])
def test_mmvq_tile_route_keeps_large_block_sums_exact(qtype, kind):
    """Activations with a common sign give q8_1 block sums far from zero (up to 32 * 127 = 4064 in magnitude, odd ones
    included), which a half cannot hold exactly beyond 2048.  The offset term of Q4_K / Q5_K on the GEMV operator is
    dmin * m * d8 * sum(q8) in exact integer arithmetic (vecdotq.cuh:328-351), so the tile route for five rows or more
    must carry the sum as an integer: fp32 results within 1e-5 of the GEMV oracle, as for centred activations."""
    ops = _ops()
    rng = np.random.default_rng(1700 + qtype)
    n, k = 2048, 4096
    w = o.make_weights(rng, qtype, n, k)
    wd = _to_dev(w)
    for m in (5, 16, 32):
        base = rng.standard_normal((m, k)).astype(np.float32)
        x32 = {"offset": 1.0 + 0.3 * base, "positive": np.abs(base) + 0.5, "negative": -np.abs(base) - 0.5}[kind].astype(np.float32)
        q = o.quantize_q8_1(x32)[0]
        sums = np.abs(np.asarray(q, dtype=np.int64).reshape(m, -1, 32).sum(-1))
        assert (sums > 2048).any() and (sums[sums > 2048] % 2 == 1).any()        # the case a half would round
        y = ops.ggml_mul_mat_vec_a8(wd, torch.from_numpy(x32).cuda(), qtype, n)
        want = o.mul_mat_a8(w, x32, qtype, n, "mmvq")
        assert o.rel_l2(y.cpu().numpy(), want) <= 1e-5, (o.TYPE_NAMES[qtype], kind, m)


def test_empty_batches_single_rows_and_rows_beyond_the_streaming_kernel():
    """The corners of the two dense operators: no rows of X at all (the reference's callers answer an empty batch
    themselves, linear.py:36-37; the operators return an empty result), a matrix of one, three and seven rows, and
    rows of 33792 to 65536 values, longer than the streaming kernel takes -- for both offset-term semantics."""
    ops = _ops()
    rng = np.random.default_rng(2900)
    w = _to_dev(o.make_weights(rng, o.Q4_K, 64, 512))
    for f in (ops.ggml_mul_mat_vec_a8, ops.ggml_mul_mat_a8):
        y = f(w, torch.empty(0, 512, dtype=torch.float16, device="cuda"), o.Q4_K, 64)
        assert y.shape == (0, 64) and y.dtype == torch.float16
    we = _to_dev(np.stack([o.make_weights(rng, o.Q4_0, 64, 256) for _ in range(4)]))
    y = ops.ggml_moe_a8_vec(torch.empty(0, 256, dtype=torch.float16, device="cuda"), we,
                            torch.empty(0, 2, dtype=torch.int32, device="cuda"), 2, o.Q4_0, 64, 0)
    assert y.shape == (0, 64)
    for qtype in (o.Q4_K, o.Q8_0, o.Q6_K, o.IQ4_XS):
        for n, k in [(1, 4096), (3, 40960), (7, 65536), (130, 33792)]:
            wn = o.make_weights(rng, qtype, n, k)
            wd = _to_dev(wn)
            for m in (1, 2, 5):
                x = rng.standard_normal((m, k)).astype(np.float32)
                xd = torch.from_numpy(x).cuda()
                err = o.rel_l2(ops.ggml_mul_mat_vec_a8(wd, xd, qtype, n).cpu().numpy(), o.mul_mat_a8(wn, x, qtype, n, "mmvq"))
                assert err <= 1e-5, (o.TYPE_NAMES[qtype], n, k, m, err)
                err = o.rel_l2(ops.ggml_mul_mat_a8(wd, xd, qtype, n).cpu().numpy(), o.mul_mat_a8(wn, x, qtype, n, "mmq"))
                assert err <= 1e-5, (o.TYPE_NAMES[qtype], n, k, m, err)


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q4_0, o.Q6_K, o.Q8_0, o.IQ2_XXS])
def test_rows_of_zeros_and_rows_at_the_bottom_of_the_float_range(qtype):
    """Activation rows that are all zero (d = 0: every code 0, the result exactly 0, no NaN from 0 / 0), rows with whole
    blocks of zeros, and a row scaled to 1e-30 (its q8_1 scales are subnormal as halves or flush to zero, as in the
    reference), at the row counts of every kernel of both dense operators."""
    ops = _ops()
    rng = np.random.default_rng(3100 + qtype)
    n, k = 96, 2048
    wn = o.make_weights(rng, qtype, n, k)
    wd = _to_dev(wn)
    for m in (1, 3, 8, 40, 200):
        x = rng.standard_normal((m, k)).astype(np.float32)
        x[0] = 0.0
        if m > 2:
            x[2, :64] = 0.0
            x[1] *= 1e-30
        for f, mode in ((ops.ggml_mul_mat_vec_a8, "mmvq"), (ops.ggml_mul_mat_a8, "mmq")):
            y = f(wd, torch.from_numpy(x).cuda(), qtype, n).cpu().numpy()
            want = o.mul_mat_a8(wn, x, qtype, n, mode)
            assert np.isfinite(y).all() and (y[0] == 0).all(), (o.TYPE_NAMES[qtype], m, mode)
            rows = [i for i in range(m) if i != 1 or m <= 2]
            assert o.rel_l2(y[rows], want[rows]) <= 1e-5, (o.TYPE_NAMES[qtype], m, mode)
            if m > 2:
                assert np.abs(y[1] - want[1]).max() <= 1e-5 * np.abs(want[1]).max() + 1e-38, (o.TYPE_NAMES[qtype], m, mode)


SPAN_TYPES = [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ4_NL]


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("qtype", SPAN_TYPES)
def test_mmvq_rows_of_whole_spans_through_lds(qtype, dt):
    """One or two rows of X over a matrix whose rows are whole 16-byte pieces at 16-byte aligned addresses: a wave fetches
    its 2048-value stretch of a row as 16-byte pieces, every byte once, and the lanes cut their blocks out of a copy in LDS
    (at 2-byte alignment for the 18-, 22-, 34-, 110- and 210-byte blocks).  Shards whose rows are a wider pitch apart
    take the same route when pitch and address are multiples of 16; when they are not, Q3_K and Q6_K (whose rows are
    whole pieces only for K a multiple of 2048) fetch the pieces from the 16-byte boundary below each stretch and the
    others load per lane; all must agree with the GEMV oracle."""
    ops = _ops()
    rng = np.random.default_rng(1700 + qtype)
    tol = 1e-5 if dt == "f32" else 1e-3
    # one, two, three waves per row; then rows whose last wave has 48, 32 or 16 of its 64 blocks (a shorter last stretch),
    # for the formats whose rows still are whole 16-byte pieces
    for n, k in [(4608, 2048), (2400, 4096), (1300, 6144), (2400, 3584), (1500, 5120), (5000, 1024), (1536, 2560)]:
        w = o.make_weights(rng, qtype, n, k)
        wd = _to_dev(w)
        for m in (1, 2, 3, 4) if qtype == o.Q8_0 else (1, 2):   # (Q8_0 fetches whole pieces up to four rows of X)
            xd, xv = _x(rng, m, k, dt)
            y = ops.ggml_mul_mat_vec_a8(wd, xd, qtype, n)
            assert o.rel_l2(y.float().cpu().numpy(), o.mul_mat_a8(w, xv, qtype, n, "mmvq")) <= tol, (o.TYPE_NAMES[qtype], n, k, m)
    # a shard inside a wider tensor: rows `extra` bytes further apart, starting `lead` bytes in
    n, k = 2400, 4096
    w = o.make_weights(rng, qtype, n, k)
    xd, xv = _x(rng, 1, k, dt)
    want = o.mul_mat_a8(w, xv, qtype, n, "mmvq")
    for lead, extra in [(32, 48), (6, 48), (32, 10)]:
        wide = torch.zeros((n, lead + w.shape[1] + extra), dtype=torch.uint8, device="cuda")
        wide[:, lead:lead + w.shape[1]] = _to_dev(w)
        y = ops.ggml_mul_mat_vec_a8(wide[:, lead:lead + w.shape[1]], xd, qtype, n)
        assert o.rel_l2(y.float().cpu().numpy(), want) <= tol, (o.TYPE_NAMES[qtype], lead, extra)


@pytest.mark.parametrize("qtype", ALL)
def test_mmvq_rows_handed_out_to_half_waves(qtype):
    """One row of X over rows of 32, 80 or 160 units (K = 1024, 2560, 5120): a row takes one, three or five half-waves of
    32 lanes, so the kernel hands rows out to half-waves (32, 10 or 6 rows side by side in a 16-wave workgroup) -- unless
    the format fetches such rows as whole 16-byte pieces, which comes first.  Both must agree with the GEMV oracle."""
    ops = _ops()
    rng = np.random.default_rng(1800 + qtype)
    for n, k in [(3000, 1024), (9000, 1024), (2600, 2560), (1700, 5120), (5200, 5120)]:   # (the first is too small: whole waves)
        w = o.make_weights(rng, qtype, n, k)
        xd, xv = _x(rng, 1, k, "f32")
        y = ops.ggml_mul_mat_vec_a8(_to_dev(w), xd, qtype, n)
        assert o.rel_l2(y.float().cpu().numpy(), o.mul_mat_a8(w, xv, qtype, n, "mmvq")) <= 1e-5, (o.TYPE_NAMES[qtype], n, k)


def test_empty_and_errors():
    ops = _ops()
    rng = np.random.default_rng(3)
    w = _to_dev(o.make_weights(rng, o.Q8_0, 8, 64))
    y = ops.ggml_mul_mat_vec_a8(w, torch.empty((0, 64), dtype=torch.float16, device="cuda"), o.Q8_0, 8)
    assert y.shape == (0, 8)
    with pytest.raises(NotImplementedError):
        ops.ggml_mul_mat_vec_a8(w, torch.zeros((1, 64), dtype=torch.float16, device="cuda"), 99, 8)
    with pytest.raises(ValueError):
        ops.ggml_mul_mat_vec_a8(w, torch.zeros((1, 64), dtype=torch.float64, device="cuda"), o.Q8_0, 8)
    with pytest.raises(ValueError):
        ops.ggml_dequantize(w, o.Q4_K, 8, 40, None)  # 320 elements is not a multiple of the 256-element block
