"""GPU parity: MMQ (int8-MFMA and half-MFMA engines), grouped MoE MMQ and per-pair MoE GEMV against the CPU oracle
(C ABI path)."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as o

pytestmark = pytest.mark.gpu

SIX = [o.Q4_0, o.Q8_0, o.Q4_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS]
MMQ_TYPES = [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS]
ALL = [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ2_XXS, o.IQ2_XS, o.IQ3_XXS,
       o.IQ1_S, o.IQ4_NL, o.IQ3_S, o.IQ2_S, o.IQ4_XS, o.IQ1_M]
HALF_ENGINE_TYPES = [o.Q4_0, o.Q5_0, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS]
TORCH_DT = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}


def _ops():
    from vllm_gguf_plugin_prism_amd import ops
    return ops


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _x(rng, m, k, dt):
    t = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(TORCH_DT[dt])
    return t.cuda(), t.to(torch.float32).numpy()


@pytest.mark.parametrize("qtype", MMQ_TYPES)
@pytest.mark.parametrize("m", [7, 83, 128, 200])
def test_mmq_matches_a8_oracle_fp32(qtype, m):
    ops = _ops()
    rng = np.random.default_rng(400 + qtype * 16 + m)
    qk = o.QUANT_SIZES[qtype][0]
    for n, k in [(256, 1024), (77, 768), (130, 736 if qk == 32 else 1280)]:
        w = o.make_weights(rng, qtype, n, k)
        xd, xv = _x(rng, m, k, "f32")
        y = ops.ggml_mul_mat_a8(_dev(w), xd, qtype, n)
        assert y.shape == (m, n) and y.dtype == torch.float32
        exp = o.mul_mat_a8(w, xv, qtype, n, "mmq")
        err = o.rel_l2(y.cpu().numpy(), exp)
        assert err <= 1e-5, (o.TYPE_NAMES[qtype], m, n, k, err)


@pytest.mark.parametrize("kind", ["offset", "positive"])
@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q2_K, o.Q4_K, o.Q5_K])
def test_tile_operators_with_activations_of_one_sign(qtype, kind):
    """The formats with an offset term on activations that share a sign: their q8_1 block sums are far from zero (up to
    32 * 127 in magnitude), so the offset term is as large as the product term and partly cancels it -- the case in which
    a block sum carried with too few bits shows.  The tile operator at the row counts of each of its kernels (streaming
    GEMV with tile sums, packed-block rows, 16-row tiles, the pipelined engine on 64-, 128- and 256-row tiles) and the
    grouped MoE operator on 16- and 32-slot blocks, fp32 results within 1e-5 of the a8 oracle as for centred activations."""
    ops = _ops()
    rng = np.random.default_rng(4300 + qtype)
    n, k = 384, 2048

    def draw(rows):
        base = rng.standard_normal((rows, k)).astype(np.float32)
        return ((1.0 + 0.3 * base) if kind == "offset" else (np.abs(base) + 0.5)).astype(np.float32)

    w = o.make_weights(rng, qtype, n, k)
    wd = _dev(w)
    for m in (3, 8, 16, 32, 64, 128, 300, 512):
        x32 = draw(m)
        if m == 3:
            sums = np.abs(np.asarray(o.quantize_q8_1(x32)[0], dtype=np.int64).reshape(m, -1, 32).sum(-1))
            assert (sums > 2048).any()
        y = ops.ggml_mul_mat_a8(wd, torch.from_numpy(x32).cuda(), qtype, n)
        err = o.rel_l2(y.cpu().numpy(), o.mul_mat_a8(w, x32, qtype, n, "mmq"))
        assert err <= 1e-5, (o.TYPE_NAMES[qtype], kind, m, err)
    e, top_k = 6, 2
    we = np.stack([o.make_weights(rng, qtype, 160, k) for _ in range(e)])
    for t in (20, 150):                       # about 7 and 50 pairs per expert: 16-slot blocks where the format has them, else 32
        x32 = draw(t)
        ids, _ = _routing(rng, t, e, top_k)
        blk = ops.moe_block_size_for(qtype, t * top_k, e)
        s_, eids, npost = o.moe_align_block_size(ids, blk, e)
        y = ops.ggml_moe_a8(torch.from_numpy(x32).cuda(), _dev(we), _dev(s_), _dev(eids), _dev(npost), qtype, 160, top_k, t, block_size=blk)
        err = o.rel_l2(y.cpu().numpy(), o.moe_a8(x32, we, s_, eids, npost, qtype, 160, top_k, t, blk))
        assert err <= 1e-5, (o.TYPE_NAMES[qtype], kind, "moe", t, blk, err)
        yv = ops.ggml_moe_a8_vec(torch.from_numpy(x32).cuda(), _dev(we), _dev(ids), top_k, qtype, 160, t)
        err = o.rel_l2(yv.cpu().numpy(), o.moe_a8_vec(x32, we, ids, top_k, qtype, 160, t))
        assert err <= 1e-5, (o.TYPE_NAMES[qtype], kind, "moe vec", t, err)


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q5_0, o.Q5_1, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K])
def test_mmq_2048_tokens_as_the_reference_tests_them(qtype):
    """The largest batch of the reference's test_mmq (tests/test_kernels.py:150-196: 7, 83, 128, 2048 tokens on
    hidden sizes 256 and 1024), here against the a8 oracle instead of gguf-py: fp32 through the integer engine,
    fp16 through the library's choice."""
    ops = _ops()
    rng = np.random.default_rng(480 + qtype)
    m = 2048
    for n, k in [(256, 1024), (1024, 256)]:
        w = o.make_weights(rng, qtype, n, k)
        wd = _dev(w)
        xd, xv = _x(rng, m, k, "f32")
        exp = o.mul_mat_a8(w, xv, qtype, n, "mmq")
        assert o.rel_l2(ops.ggml_mul_mat_a8(wd, xd, qtype, n).cpu().numpy(), exp) <= 1e-5
        xh, xhv = _x(rng, m, k, "f16")
        y = ops.ggml_mul_mat_a8(wd, xh, qtype, n)
        assert y.shape == (m, n) and y.dtype == torch.float16
        assert o.rel_l2(y.float().cpu().numpy(), o.mul_mat_a8(w, xhv, qtype, n, "mmq")) <= 1e-3


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("qtype", MMQ_TYPES)
def test_mmq_handful_of_rows_keeps_tile_semantics(qtype, dt):
    """Up to eight rows of X run on the streaming GEMV kernel.  The operator is still the tile GEMM: Q4_K / Q5_K take
    their offset from the stored block sums and Q5_0 from the quant sums, which is where the reference's two operators
    part (the oracle's "mmq" and "mmvq" results differ by 1e-2 .. 1e-4 on these weights)."""
    ops = _ops()
    rng = np.random.default_rng(450 + qtype)
    n, k = 200, 1536
    w = o.make_weights(rng, qtype, n, k)
    wd = _dev(w)
    for m in (1, 2, 3, 4, 5, 6, 8):
        xd, xv = _x(rng, m, k, dt)
        y = ops.ggml_mul_mat_a8(wd, xd, qtype, n)
        assert y.shape == (m, n) and y.dtype == TORCH_DT[dt]
        err = o.rel_l2(y.float().cpu().numpy(), o.mul_mat_a8(w, xv, qtype, n, "mmq"))
        assert err <= (1e-5 if dt == "f32" else 1e-3), (o.TYPE_NAMES[qtype], m, err)
        # the engines asked for by name are still the tile kernels
        if dt == "f16":
            yi = ops.ggml_mul_mat_a8(wd, xd, qtype, n, engine="int8")
            assert o.rel_l2(yi.float().cpu().numpy(), y.float().cpu().numpy()) <= 1e-3


@pytest.mark.parametrize("engine", ["auto", "int8", "half"])
@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("qtype", MMQ_TYPES)
def test_mmq_half_outputs_within_tolerance(qtype, dt, engine):
    # stated tolerance vs the a8 oracle: rel-L2 <= 1e-3 for fp16 outputs, 4e-3 for bf16 (8-bit significand); it holds
    # for both arithmetic engines ("auto" is the half-MFMA engine wherever that one applies)
    if engine == "half" and qtype not in HALF_ENGINE_TYPES:
        pytest.skip("no half-MFMA engine for this format")
    ops = _ops()
    rng = np.random.default_rng(500 + qtype)
    n, k = 384, 2048
    w = o.make_weights(rng, qtype, n, k)
    for m in (160, 7):
        xd, xv = _x(rng, m, k, dt)
        y = ops.ggml_mul_mat_a8(_dev(w), xd, qtype, n, engine=engine).to(torch.float32).cpu().numpy()
        assert o.rel_l2(y, o.mul_mat_a8(w, xv, qtype, n, "mmq")) <= (1e-3 if dt == "f16" else 4e-3)
        assert o.rel_l2(y, o.mul_mat_f32(w, xv, qtype, n)) <= 2e-2


def test_mmq_engines_differ_only_by_operand_rounding():
    # both engines against the same fp32-output run of the integer engine: the half engine adds the rounding of its
    # two operands to half precision (about 3.5e-4) to the rounding of the fp16 result (2.1e-4) and nothing else
    ops = _ops()
    rng = np.random.default_rng(77)
    for qtype in HALF_ENGINE_TYPES:
        n, k, m = 320, 2048, 96
        w = _dev(o.make_weights(rng, qtype, n, k))
        xd, _ = _x(rng, m, k, "f16")
        exact = ops.ggml_mul_mat_a8(w, xd.float(), qtype, n).double()
        half = ops.ggml_mul_mat_a8(w, xd, qtype, n, engine="half").double()
        int8 = ops.ggml_mul_mat_a8(w, xd, qtype, n, engine="int8").double()
        e_half = float((half - exact).norm() / exact.norm()), float((int8 - exact).norm() / exact.norm())
        assert e_half[1] <= 3e-4 and e_half[0] <= 6e-4, (o.TYPE_NAMES[qtype], e_half)


@pytest.mark.parametrize("qtype", [o.Q6_K, o.Q4_K, o.Q4_0, o.Q2_K, o.Q8_0])
@pytest.mark.parametrize("m,n", [(512, 12800), (256, 12800), (256, 6400), (300, 200)])
def test_mmq_half_engine_every_tile_configuration(qtype, m, n):
    """The half-MFMA launcher takes the largest of 256x128, 128x128, 128x64 and 64x64 tiles that still yields 180
    workgroups.  One shape per regime with ragged M and N edges; K is not a multiple of the 64-element step for the
    32-element formats, so the last step is half empty and the offset pass ends inside a group of eight blocks."""
    ops = _ops()
    rng = np.random.default_rng(1100 + qtype + m)
    k = 256 if o.QUANT_SIZES[qtype][0] == 256 else 352
    w = o.make_weights(rng, qtype, n - 3, k)
    xd, xv = _x(rng, m - 5, k, "f16")
    y = ops.ggml_mul_mat_a8(_dev(w), xd, qtype, n - 3, engine="half")
    assert y.shape == (m - 5, n - 3) and y.dtype == torch.float16
    assert o.rel_l2(y.float().cpu().numpy(), o.mul_mat_a8(w, xv, qtype, n - 3, "mmq")) <= 1e-3


@pytest.mark.parametrize("qtype", [o.Q6_K, o.Q4_K, o.Q4_0])
@pytest.mark.parametrize("m", [200, 100])
def test_mmq_half_engine_split_k(qtype, m):
    """Few output tiles and a long K: the half engine splits K over several workgroups per tile (fp32 partial tiles in
    the workspace, summed by a second launch) when the workspace is sized by gguf_mmq_workspace_bytes, and must not
    when it has only the minimum.  Same tolerance either way; the offset pass belongs to the first split."""
    from vllm_gguf_plugin_prism_amd import _lib
    ops = _ops()
    rng = np.random.default_rng(1300 + qtype + m)
    n, k = 250, 4096
    assert _lib.lib().gguf_mmq_workspace_bytes(m, n, k) > m * _lib.lib().gguf_q8_1_row_bytes(k) + 256   # room for partials
    w = o.make_weights(rng, qtype, n, k)
    xd, xv = _x(rng, m, k, "f16")
    exp = o.mul_mat_a8(w, xv, qtype, n, "mmq")
    y_split = ops.ggml_mul_mat_a8(_dev(w), xd, qtype, n, engine="half")
    assert o.rel_l2(y_split.float().cpu().numpy(), exp) <= 1e-3
    # the plain C entry point passes no workspace size: no split
    ws = torch.empty(m * _lib.lib().gguf_q8_1_row_bytes(k), dtype=torch.uint8, device="cuda")
    y_plain = torch.empty_like(y_split)
    wd = _dev(w)
    rc = _lib.lib().gguf_mmq(wd.data_ptr(), xd.data_ptr(), 1, ws.data_ptr(), y_plain.data_ptr(), qtype, n, k, m,
                             torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert o.rel_l2(y_plain.float().cpu().numpy(), exp) <= 1e-3
    assert o.rel_l2(y_plain.float().cpu().numpy(), y_split.float().cpu().numpy()) <= 5e-4   # fp32 sums in another order, rounded to half


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("qtype", MMQ_TYPES)
def test_dequant_gemm_is_the_dense_product(qtype, dt):
    """ggml_dequant_gemm = x @ ggml_dequantize(W).T with unquantized activations (the reference's fallback path,
    linear.py:50-58) in one kernel.  Against the product formed in fp32 from the library's own bit-exact half-precision
    dequantization, what remains is the rounding of the result (2.1e-4 for fp16) and, for formats whose scale product the
    kernel rounds before the code is applied, one more half rounding of the weight (bf16 activations add nothing: they
    are half-representable in this range); against the fp32 oracle the half-precision weights show as well."""
    ops = _ops()
    rng = np.random.default_rng(1500 + qtype)
    qk = o.QUANT_SIZES[qtype][0]
    for m, n, k in [(160, 384, 2048), (7, 130, 736 if qk == 32 else 768), (300, 6400, 256 if qk == 256 else 352)]:
        w = o.make_weights(rng, qtype, n, k)
        wd = _dev(w)
        xd, xv = _x(rng, m, k, dt)
        y = ops.ggml_dequant_gemm(wd, xd, qtype, n)
        assert y.shape == (m, n) and y.dtype == TORCH_DT[dt]
        dense = ops.ggml_dequantize(wd, qtype, n, k, torch.float16).float()
        ref = (xd.float() @ dense.T).cpu().numpy()
        got = y.float().cpu().numpy()
        assert o.rel_l2(got, ref) <= (6e-4 if dt == "f16" else 3e-3), (o.TYPE_NAMES[qtype], m, n, k, o.rel_l2(got, ref))
        assert o.rel_l2(got, o.mul_mat_f32(w, xv, qtype, n)) <= (1e-3 if dt == "f16" else 4e-3)


def test_dequant_gemm_split_k_and_rejections():
    ops = _ops()
    rng = np.random.default_rng(1600)
    m, n, k = 200, 250, 4096                      # few tiles, long K: the K split engages
    w = o.make_weights(rng, o.IQ2_XXS, n, k)
    xd, xv = _x(rng, m, k, "f16")
    y = ops.ggml_dequant_gemm(_dev(w), xd, o.IQ2_XXS, n)
    assert o.rel_l2(y.float().cpu().numpy(), o.mul_mat_f32(w, xv, o.IQ2_XXS, n)) <= 1e-3
    x32, _ = _x(rng, 4, 256, "f32")
    w6 = _dev(o.make_weights(rng, o.Q6_K, 64, 256))
    with pytest.raises(ValueError):
        ops.ggml_dequant_gemm(w6, x32, o.Q6_K, 64)
    wi = _dev(o.make_weights(rng, o.IQ3_S, 64, 256))
    with pytest.raises(NotImplementedError):
        ops.ggml_dequant_gemm(wi, xd[:4, :256].contiguous(), o.IQ3_S, 64)


def test_mmq_half_engine_splits_the_last_round():
    """More tiles than the chip holds at once and a sparse last round (296 tiles of 256x128 on 256 CUs): the 40 tiles of
    that round are split along K and summed from fp32 partial tiles; the other 256 are whole.  Both kinds must agree
    with the integer engine, and the result must not depend on whether the workspace had room for the split."""
    from vllm_gguf_plugin_prism_amd import _lib
    ops = _ops()
    rng = np.random.default_rng(1700)
    m, n, k = 512, 18944, 1024
    w = _dev(np.concatenate([o.make_weights(rng, o.Q6_K, 2368, k) for _ in range(8)], axis=0))
    xd, _ = _x(rng, m, k, "f16")
    assert _lib.lib().gguf_mmq_workspace_bytes(m, n, k) > m * _lib.lib().gguf_q8_1_row_bytes(k) + 256
    y = ops.ggml_mul_mat_a8(w, xd, o.Q6_K, n, engine="half").float()
    ref = ops.ggml_mul_mat_a8(w, xd.float(), o.Q6_K, n).double()          # integer engine, fp32 result
    err = ((y.double() - ref).norm(dim=0) / ref.norm(dim=0))               # per output column: every tile is looked at
    assert float(err.max()) <= 1.5e-3 and float((y.double() - ref).norm() / ref.norm()) <= 6e-4
    # the half engine's row region and nothing behind it: no room for partial tiles, no split
    kp = (k + 511) // 512 * 512
    ws = torch.empty(m * (_lib.lib().gguf_q8_1_row_bytes(k) + 2 * (kp + 128)), dtype=torch.uint8, device="cuda")
    y_plain = torch.empty_like(y, dtype=torch.float16)
    rc = _lib.lib().gguf_mmq_engine(w.data_ptr(), xd.data_ptr(), 1, ws.data_ptr(), y_plain.data_ptr(), o.Q6_K, n, k, m,
                                    ops.MMQ_ENGINES["half"], ws.numel(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    # a workspace that holds the quantized rows only is too small for this engine, and says so
    rc = _lib.lib().gguf_mmq_engine(w.data_ptr(), xd.data_ptr(), 1, ws.data_ptr(), y_plain.data_ptr(), o.Q6_K, n, k, m,
                                    ops.MMQ_ENGINES["half"], m * _lib.lib().gguf_q8_1_row_bytes(k), torch.cuda.current_stream().cuda_stream)
    assert rc == -6
    assert float((y_plain.double() - y.double()).norm() / ref.norm()) <= 4e-4


def test_mmq_engine_rejections():
    ops = _ops()
    rng = np.random.default_rng(5)
    w = _dev(o.make_weights(rng, o.Q4_1, 64, 256))
    x16, _ = _x(rng, 4, 256, "f16")
    x32, _ = _x(rng, 4, 256, "f32")
    with pytest.raises(NotImplementedError):
        ops.ggml_mul_mat_a8(w, x16, o.Q4_1, 64, engine="half")       # Q4_1 keeps the reference's half-rounded scale products
    w6 = _dev(o.make_weights(rng, o.Q6_K, 64, 256))
    with pytest.raises(ValueError):
        ops.ggml_mul_mat_a8(w6, x32, o.Q6_K, 64, engine="half")      # fp32 results stay on the integer engine
    assert ops.ggml_mul_mat_a8(w6, x32, o.Q6_K, 64).dtype == torch.float32


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_K, o.Q6_K, o.Q2_K, o.Q5_1])
@pytest.mark.parametrize("m,n", [(512, 12800), (128, 16640), (300, 200)])
def test_mmq_every_tile_configuration(qtype, m, n):
    """The launcher picks its tile by output-tile count: 128x128 (>= 400 large tiles), 64x64 (more than 512 small
    tiles) or 64x64 with the step's blocks split over two wave sets.  One shape per regime, ragged edges included."""
    ops = _ops()
    rng = np.random.default_rng(1000 + qtype + m)
    k = 256
    w = o.make_weights(rng, qtype, n, k)
    xd, xv = _x(rng, m, k, "f32")
    y = ops.ggml_mul_mat_a8(_dev(w), xd, qtype, n)
    exp = o.mul_mat_a8(w, xv, qtype, n, "mmq")
    assert o.rel_l2(y.cpu().numpy(), exp) <= 1e-5


def test_mmq_and_mmvq_agree():
    # same contraction through both paths; Q4_K differs only by which block sum the offset term uses
    ops = _ops()
    rng = np.random.default_rng(600)
    for qtype in SIX:
        w = _dev(o.make_weights(rng, qtype, 128, 1024))
        xd, _ = _x(rng, 5, 1024, "f32")
        a = ops.ggml_mul_mat_a8(w, xd, qtype, 128).cpu().numpy()
        b = ops.ggml_mul_mat_vec_a8(w, xd, qtype, 128).cpu().numpy()
        assert o.rel_l2(a, b) <= (2e-2 if qtype == o.Q4_K else 1e-5), o.TYPE_NAMES[qtype]


@pytest.mark.parametrize("m", [128, 512, 2048])
def test_config3_q6_k_qwen_mlp_slices(m):
    # Qwen2.5-7B MLP shapes at full K; N is cut to 1024 rows so the fp64 oracle stays in seconds
    ops = _ops()
    rng = np.random.default_rng(3)
    for n, k in [(1024, 3584), (1024, 18944)]:
        w = o.make_weights(rng, o.Q6_K, n, k)
        xd, xv = _x(rng, m, k, "f16")
        y = ops.ggml_mul_mat_a8(_dev(w), xd, o.Q6_K, n).to(torch.float32).cpu().numpy()
        assert o.rel_l2(y, o.mul_mat_a8(w, xv, o.Q6_K, n, "mmq")) <= 1e-3


@pytest.mark.parametrize("engine", ["auto", "half"])
@pytest.mark.parametrize("m", [128, 512, 2048])
@pytest.mark.parametrize("n,k", [(18944, 3584), (3584, 18944)])
def test_config3_q6_k_full_size(n, k, m, engine):
    """Config 3 at its real shapes, with the tile plans the benchmark times: whole tiles, the tiles of a sparse last
    round split along K ([18944,3584] at M = 512: rows from 16384 on; at M = 2048: rows from 18432 on) and outputs
    with too few tiles for the chip, every tile split ([3584,18944]).  The fp64 oracle checks a sample of weight rows
    over all token rows, chosen to fall into each of those groups; doubling the activations must double every result
    exactly, which looks at the whole output."""
    from vllm_gguf_plugin_prism_amd import synth
    ops = _ops()
    rng = np.random.default_rng(31 + m + n)
    w = synth.random_blocks(rng, o.Q6_K, n, k)       # raw valid blocks, d ~ U(1e-4, 1e-2): a numpy quantizer at this size takes a minute
    x = rng.standard_normal((m, k)).astype(np.float16)
    wd, xd = _dev(w), torch.from_numpy(x).cuda()
    y = ops.ggml_mul_mat_a8(wd, xd, o.Q6_K, n, engine=engine)
    assert y.shape == (m, n) and y.dtype == torch.float16
    marks = [0, 64, 16384 - 32, 16384, 18432 - 32, 18432]
    rows = np.unique(np.concatenate([np.arange(a, a + 40) for a in marks if a + 40 <= n] + [np.arange(n - 70, n), rng.integers(0, n, 24)]))
    want = o.mul_mat_a8(w[rows], x.astype(np.float32), o.Q6_K, len(rows), "mmq")
    assert o.rel_l2(y[:, torch.from_numpy(rows).cuda()].float().cpu().numpy(), want) <= 1e-3
    y2 = ops.ggml_mul_mat_a8(wd, xd * 2, o.Q6_K, n, engine=engine)
    if engine == "auto":
        normal = y.abs() >= 2.0 ** -13          # a result in the half subnormals has fewer bits than its double
        assert torch.equal(y2[normal], (y * 2)[normal])
        assert o.rel_l2(y2.float().cpu().numpy(), 2 * y.float().cpu().numpy()) <= 1e-6
    else:   # the half engine rounds d8 * q to half: doubling keeps that exact too, short of overflow
        assert o.rel_l2(y2.float().cpu().numpy(), 2 * y.float().cpu().numpy()) <= 1e-3


def _routing(rng, t, e, top_k):
    logits = rng.standard_normal((t, e)).astype(np.float32)
    ids = np.argsort(-logits, axis=1)[:, :top_k].astype(np.int32)
    sel = np.take_along_axis(logits, ids.astype(np.int64), axis=1)
    wts = np.exp(sel - sel.max(axis=1, keepdims=True))
    return ids, (wts / wts.sum(axis=1, keepdims=True)).astype(np.float32)


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K])
@pytest.mark.parametrize("t,top_k,e", [(7, 2, 8), (83, 4, 16), (128, 8, 64)])
def test_moe_grouped_matches_oracle(qtype, t, top_k, e):
    ops = _ops()
    rng = np.random.default_rng(700 + qtype + t)
    n, k = 160, 512
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    xd, xv = _x(rng, t, k, "f32")
    ids, _ = _routing(rng, t, e, top_k)
    blk = ops.ggml_moe_get_block_size(qtype)
    assert blk > 0
    s, eids, npost = o.moe_align_block_size(ids, blk, e)
    y = ops.ggml_moe_a8(xd, _dev(w), _dev(s), _dev(eids), _dev(npost), qtype, n, top_k, t)
    assert y.shape == (t * top_k, n)
    exp = o.moe_a8(xv, w, s, eids, npost, qtype, n, top_k, t, blk)
    assert o.rel_l2(y.cpu().numpy(), exp) <= 1e-5
    # second stage of the pipeline: top_k = 1 over tokens * top_k rows, same sorted ids
    x2d, x2v = _x(rng, t * top_k, k, "f32")
    y2 = ops.ggml_moe_a8(x2d, _dev(w), _dev(s), _dev(eids), _dev(npost), qtype, n, 1, t * top_k)
    exp2 = o.moe_a8(x2v, w, s, eids, npost, qtype, n, 1, t * top_k, blk)
    assert o.rel_l2(y2.cpu().numpy(), exp2) <= 1e-5


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q8_0, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS])
@pytest.mark.parametrize("t,top_k,e", [(7, 2, 8), (83, 4, 32), (100, 8, 64)])
def test_moe_grouped_blocks_of_16_slots(qtype, t, top_k, e):
    """The grouped operator on a routing sorted with blocks of 16 slots (ggml_moe_a8(..., block_size=16)): the tile
    operator's arithmetic (stored block sums for the offset terms of Q4_K / Q5_K) on 16-row tiles, both stages of the
    layer, against the oracle's per-pair definition; rows that no slot names stay zero."""
    ops = _ops()
    rng = np.random.default_rng(740 + qtype + t)
    n, k = 160, 512
    assert ops.moe_block_size_for(qtype, t * top_k, e) == (16 if t * top_k <= 12 * e else 32)
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    xd, xv = _x(rng, t, k, "f32")
    ids, _ = _routing(rng, t, e, top_k)
    s, eids, npost = o.moe_align_block_size(ids, 16, e)
    y = ops.ggml_moe_a8(xd, _dev(w), _dev(s), _dev(eids), _dev(npost), qtype, n, top_k, t, block_size=16)
    assert o.rel_l2(y.cpu().numpy(), o.moe_a8(xv, w, s, eids, npost, qtype, n, top_k, t, 16)) <= 1e-5
    x2d, x2v = _x(rng, t * top_k, k, "f32")
    y2 = ops.ggml_moe_a8(x2d, _dev(w), _dev(s), _dev(eids), _dev(npost), qtype, n, 1, t * top_k, block_size=16)
    assert o.rel_l2(y2.cpu().numpy(), o.moe_a8(x2v, w, s, eids, npost, qtype, n, 1, t * top_k, 16)) <= 1e-5
    # a routing that leaves pairs out: their rows are zero
    s2 = s.copy()
    dropped = s2[:16][s2[:16] < t * top_k]
    s2[:16] = t * top_k
    y3 = ops.ggml_moe_a8(xd, _dev(w), _dev(s2), _dev(eids), _dev(npost), qtype, n, top_k, t, block_size=16).cpu().numpy()
    assert np.all(y3[dropped] == 0)


def test_moe_16_slot_launch_geometry_does_not_change_results():
    """The launcher of the 16-slot tiles guesses, from the length of the sorted array and the pair count, how the blocks
    will fall into rounds of workgroups and asks for an LDS size that lets two or three of them share a CU.  That guess
    moves time only: the same routing in a sorted array with room for twice the experts (more padding slots behind
    num_tokens_post_padded, which no block reaches) lands on the other side of the estimate -- 64 experts x 16 feature
    tiles at 4 pairs per expert is the 'two per CU' case, 128 apparent experts is not -- and must give the same bits."""
    ops = _ops()
    rng = np.random.default_rng(4242)
    qtype, e, n, k, t, top_k = o.Q4_0, 64, 2048, 256, 32, 8
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    wd = _dev(w)
    xd, xv = _x(rng, t, k, "f32")
    ids, _ = _routing(rng, t, e, top_k)
    s, eids, npost = o.moe_align_block_size(ids, 16, e)
    y = ops.ggml_moe_a8(xd, wd, _dev(s), _dev(eids), _dev(npost), qtype, n, top_k, t, block_size=16)
    assert o.rel_l2(y.cpu().numpy(), o.moe_a8(xv, w, s, eids, npost, qtype, n, top_k, t, 16)) <= 1e-5
    extra = 15 * e // 16 * 16
    s_long = np.concatenate([s, np.full(extra, t * top_k, dtype=s.dtype)])
    eids_long = np.concatenate([eids, np.zeros(extra // 16, dtype=eids.dtype)])
    y_long = ops.ggml_moe_a8(xd, wd, _dev(s_long), _dev(eids_long), _dev(npost), qtype, n, top_k, t, block_size=16)
    assert torch.equal(y, y_long)


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_K])
@pytest.mark.parametrize("t,top_k", [(2048, 8), (83, 4)])
def test_moe_256_experts_as_the_reference_tests_them(qtype, t, top_k):
    """Expert count and token counts of the reference's test_moe (tests/test_kernels.py:313-361: 256 experts, top-4 and
    top-8, up to 2048 tokens), both operators, on a narrower layer so that the fp64 oracle stays in seconds."""
    ops = _ops()
    rng = np.random.default_rng(760 + qtype + t)
    e, n, k = 256, 128, 512
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    wd = _dev(w)
    xd, xv = _x(rng, t, k, "f32")
    ids, _ = _routing(rng, t, e, top_k)
    blk = ops.ggml_moe_get_block_size(qtype)
    s, eids, npost = o.moe_align_block_size(ids, blk, e)
    y = ops.ggml_moe_a8(xd, wd, _dev(s), _dev(eids), _dev(npost), qtype, n, top_k, t)
    assert o.rel_l2(y.cpu().numpy(), o.moe_a8(xv, w, s, eids, npost, qtype, n, top_k, t, blk)) <= 1e-5
    yv = ops.ggml_moe_a8_vec(xd, wd, _dev(ids), top_k, qtype, n, t)
    assert o.rel_l2(yv.cpu().numpy(), o.moe_a8_vec(xv, w, ids, top_k, qtype, n, t)) <= 1e-5


def test_more_than_256_experts_take_the_per_pair_operator():
    """The grouped kernel keeps the reference's guard on expert ids (moe.cuh:33), so the wrapper refuses a tensor of
    more than 256 experts and the layer-level dispatch sends such a layer to the per-pair operator, which has no
    limit; the result must match the per-token definition of the layer."""
    from vllm_gguf_plugin_prism_amd import dispatch as D
    ops = _ops()
    rng = np.random.default_rng(777)
    e, n, k, t, top_k, qtype = 300, 64, 256, 70, 2, o.Q8_0
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    xd, xv = _x(rng, t, k, "f32")
    ids, wts = _routing(rng, t, e, top_k)
    ids[0, 0] = 299                                    # an expert the grouped kernel would have dropped
    ids[0, 1] = 3
    blk = ops.ggml_moe_get_block_size(qtype)
    s, eids, npost = o.moe_align_block_size(ids, blk, e)
    with pytest.raises(NotImplementedError):
        ops.ggml_moe_a8(xd, _dev(w), _dev(s), _dev(eids), _dev(npost), qtype, n, top_k, t)
    yv = ops.ggml_moe_a8_vec(xd, _dev(w), _dev(ids), top_k, qtype, n, t)
    assert o.rel_l2(yv.cpu().numpy(), o.moe_a8_vec(xv, w, ids, top_k, qtype, n, t)) <= 1e-5
    assert D.select_moe_path(qtype, qtype, t) == "grouped"        # what the reference's policy says for 70 tokens
    w2 = np.stack([o.make_weights(rng, qtype, k, n // 2) for _ in range(e)])
    got = D.fused_moe_gguf(xd, _dev(w), _dev(w2), torch.from_numpy(wts).cuda(), _dev(ids), qtype, qtype, "silu")
    h = o.moe_a8_vec(xv, w, ids, top_k, qtype, n, t)
    a = o.silu_and_mul(h.astype(np.float64)).astype(np.float32)
    y = o.moe_a8_vec(a, w2, ids.reshape(-1), 1, qtype, k, t * top_k).reshape(t, top_k, k)
    want = (y * wts[:, :, None]).sum(1)
    assert o.rel_l2(got.cpu().numpy(), want) <= 1e-4


def test_moe_grouped_padding_and_bad_experts_write_nothing():
    ops = _ops()
    rng = np.random.default_rng(800)
    t, top_k, e, n, k, qtype = 20, 2, 6, 64, 256, o.Q4_0
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    xd, xv = _x(rng, t, k, "f32")
    ids, _ = _routing(rng, t, e, top_k)
    blk = ops.ggml_moe_get_block_size(qtype)
    s, eids, npost = o.moe_align_block_size(ids, blk, e)
    eids2 = eids.copy()
    eids2[0] = 300            # out-of-range expert: its block is skipped (moe.cuh:33)
    y = ops.ggml_moe_a8(xd, _dev(w), _dev(s), _dev(eids2), _dev(npost), qtype, n, top_k, t).cpu().numpy()
    exp = o.moe_a8(xv, w, s, eids2, npost, qtype, n, top_k, t, blk)
    assert o.rel_l2(y, exp) <= 1e-5
    skipped = s[:blk][s[:blk] < t * top_k]
    assert len(skipped) > 0 and np.all(y[skipped] == 0)


@pytest.mark.parametrize("t,top_k,e", [(2, 2, 8), (64, 8, 64), (33, 1, 3)])
@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_K, o.IQ2_XXS])
def test_moe_vec_grouped_and_per_pair_grids(qtype, t, top_k, e):
    """Few pairs per expert run one pair per workgroup row, many pairs are sorted by expert and run four at a time;
    both must give the per-pair result, including ragged last groups and experts nobody picked."""
    ops = _ops()
    rng = np.random.default_rng(950 + qtype + t)
    n, k = 72, 512
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    xd, xv = _x(rng, t, k, "f32")
    ids, _ = _routing(rng, t, e, top_k)
    y = ops.ggml_moe_a8_vec(xd, _dev(w), _dev(ids), top_k, qtype, n, t)
    assert o.rel_l2(y.cpu().numpy(), o.moe_a8_vec(xv, w, ids, top_k, qtype, n, t)) <= 1e-5


@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q8_0, o.Q4_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS])
def test_moe_vec_few_pairs_stream_each_expert(qtype, dt):
    """With fewer than two pairs per expert every pair walks its expert's matrix on the streaming GEMV kernel, which
    quantizes the pair's token itself: rows that are whole 2048-value spans (the staged loads of Q4_K) and shorter
    ones, an output that does not divide into the workgroups' bands, the gated activation of the layer's second GEMM
    folded into the quantisation, an expert id outside the table (left out, the others unaffected), and rows short
    enough for two of them to share a wave."""
    ops = _ops()
    rng = np.random.default_rng(1500 + qtype)
    tol = {"f32": 1e-5, "f16": 1e-3, "bf16": 8e-3}[dt]
    # (the last: rows of 32 units and bands of 66 rows, which half-waves walk in three turns where waves take five)
    for t, top_k, e, n, k in [(1, 8, 64, 200, 2048), (3, 2, 8, 77, 512), (5, 1, 16, 300, 1024), (2, 4, 8, 2100, 1024)]:
        w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
        xd, xv = _x(rng, t, k, dt)
        ids, _ = _routing(rng, t, e, top_k)
        assert t * top_k < 2 * e
        y = ops.ggml_moe_a8_vec(xd, _dev(w), _dev(ids), top_k, qtype, n, t)
        want = o.moe_a8_vec(xv, w, ids, top_k, qtype, n, t)
        assert o.rel_l2(y.float().cpu().numpy(), want) <= tol, (o.TYPE_NAMES[qtype], t, e, k)
        bad = ids.copy()
        bad[0, 0] = e + 2
        y2 = ops.ggml_moe_a8_vec(xd, _dev(w), _dev(bad), top_k, qtype, n, t)
        assert torch.equal(y2[1:], y[1:])
        # second GEMM of a layer: rows [gate | up] per pair, act(gate) * up quantized inside the kernel
        pairs = t * top_k
        h = (torch.randn(pairs, 2 * k, device="cuda") * 2).to(TORCH_DT[dt])
        sep = (torch.nn.functional.silu(h[:, :k]) * h[:, k:]).contiguous()
        flat = _dev(ids.reshape(pairs, 1))
        got = ops.ggml_moe_a8_vec(h, _dev(w), flat, 1, qtype, n, pairs, activation="silu")
        ref = o.moe_a8_vec(sep.float().cpu().numpy(), w, ids.reshape(pairs, 1), 1, qtype, n, pairs)
        # (torch's and the kernel's exp may differ in the last bit of a few activations: a quant moves by one step at most)
        assert o.rel_l2(got.float().cpu().numpy(), ref) <= max(tol, 5e-4), (o.TYPE_NAMES[qtype], "gated", t, e, k)


@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("qtype", [q for q in sorted(o.QUANT_SIZES) if q != 9])      # (9 is q8_1, the activations' format)
def test_moe_layer_in_two_launches_matches_the_separate_steps(qtype, dt):
    """moe_vec_layer (first GEMV with the activation and the q8_1 quantisation in its epilogue; second GEMV with the
    routing weights and the sum over the top-k axis) against ggml_moe_a8_vec, ggml_moe_a8_vec(..., activation=) and
    moe_weighted_sum run one by one, to fp32 rounding -- the separate steps are held to the oracle by the tests above.
    Rows of 32 units on half-waves and longer rows on waves, top-k from 1 to 8, inner sizes that leave the last band
    short, a second format for the down projection, an expert id outside the table (that pair adds nothing), and shapes
    the kernels decline."""
    ops = _ops()
    rng = np.random.default_rng(1700 + qtype)
    qk = o.QUANT_SIZES[qtype][0]
    other = o.Q8_0 if qk == 32 else o.Q4_0                 # the down projection in another format (32-value blocks)
    # tokens, top_k, experts, hidden, inner
    # (the last: 33 and 35 blocks of 32 values -- rows that end inside a wave and a last band of 32 features)
    for case, (t, top_k, e, hid, inner) in enumerate([(1, 8, 16, 2048, 1024), (3, 2, 8, 512, 768), (2, 4, 8, 1024, 2048), (5, 1, 8, 256, 1280),
                                                     (1, 2, 4, 4096, 512), (2, 3, 6, 1056, 1120)]):
        for qt2 in (qtype, other) if case < 2 else (qtype,):
            if inner % o.QUANT_SIZES[qt2][0] or hid % qk:
                continue
            w13 = np.stack([o.make_weights(rng, qtype, 2 * inner, hid) for _ in range(e)])
            w2 = np.stack([o.make_weights(rng, qt2, hid, inner) for _ in range(e)])
            w13d, w2d = _dev(w13), _dev(w2)
            ids, wts = _routing(rng, t, e, top_k)
            pairs = t * top_k
            assert ops.moe_vec_layer_takes(qtype, qt2, hid, inner, hid, top_k, t, e)
            x = torch.randn(t, hid, device="cuda")
            # (the random weights' scales are arbitrary: bring the first GEMV's results to a few units, so that the gated
            #  products stay far below the half-precision range the q8_1 scales are stored in)
            x = (x * (4.0 / ops.ggml_moe_a8_vec(x, w13d, _dev(ids), top_k, qtype, 2 * inner, t).abs().max())).to(TORCH_DT[dt])
            for bad in (False, True):
                if bad:
                    ids = ids.copy()
                    ids[0, top_k - 1] = e + 3
                h = ops.ggml_moe_a8_vec(x, w13d, _dev(ids), top_k, qtype, 2 * inner, t)
                y = ops.ggml_moe_a8_vec(h, w2d, _dev(ids.reshape(pairs, 1)), 1, qt2, hid, pairs, activation="silu")
                if bad:
                    y[top_k - 1].zero_()                   # the separate steps leave that pair's row unwritten
                want = torch.empty((t, hid), dtype=x.dtype, device="cuda")
                ops.moe_weighted_sum(y.reshape(t, top_k, hid), _dev(wts), want)
                got = ops.moe_vec_layer(x, w13d, w2d, _dev(wts), _dev(ids), qtype, qt2, "silu")
                assert not torch.isnan(want).any()
                # (Most cases agree bit for bit.  Not all: the compiler contracts multiply-adds per kernel, so a sum or an
                #  exponential may differ in its last bit and, about once in 10^5 values, move one quant of h by a step, which
                #  shifts every output of that token by about 1e-4 of its size.)
                err = o.rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy())
                assert err <= {"f32": 5e-4, "f16": 1e-3, "bf16": 4e-3}[dt], \
                    f"{o.TYPE_NAMES[qtype]} {o.TYPE_NAMES[qt2]} {dt} t={t} top_k={top_k} hid={hid} inner={inner} bad={bad} rel-L2 {err}"
    # top_k times the waves a row of the down projection takes exceed a workgroup; experts shared by several pairs each
    # when there are more of them than the tile kernels' guard on expert ids admits: declined
    assert not ops.moe_vec_layer_takes(qtype, qtype, 2048, 8192, 2048, 8, 1, 64)
    assert not ops.moe_vec_layer_takes(qtype, qtype, 256, 256, 256, 8, 200, 300)
    with pytest.raises(ValueError):
        row = 256 // qk * o.QUANT_SIZES[qtype][1]
        ops.moe_vec_layer(torch.zeros(200, 256, device="cuda", dtype=TORCH_DT[dt]), _dev(np.zeros((300, 512, row), dtype=np.uint8)),
                          _dev(np.zeros((300, 256, row), dtype=np.uint8)), _dev(np.ones((200, 8), dtype=np.float32)),
                          _dev(np.zeros((200, 8), dtype=np.int32)), qtype, qtype, "silu")


@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_1, o.Q5_1, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS])
def test_moe_layer_on_tiles_matches_the_separate_steps(qtype, dt):
    """moe_vec_layer where a few pairs share each expert: quantize and one routing sort, first GEMM on 16-slot tiles with
    the activation and the q8_1 quantisation in its epilogue, second GEMM from those rows, weighted sum -- against the
    per-pair operator called twice and moe_weighted_sum (which take the same tile kernels with a sort and a quantize
    launch more each).  Inner sizes that end inside a 128-column tile, an expert without pairs, a second format."""
    ops = _ops()
    rng = np.random.default_rng(1800 + qtype)
    qk = o.QUANT_SIZES[qtype][0]
    other = o.Q8_0 if qtype != o.Q8_0 else o.Q4_0
    for case, (t, top_k, e, hid, inner) in enumerate([(24, 4, 8, 512, 768), (40, 2, 6, 256, 1280 if qk == 32 else 1024)]):
        for qt2 in (qtype, other) if case == 0 else (qtype,):
            w13 = np.stack([o.make_weights(rng, qtype, 2 * inner, hid) for _ in range(e)])
            w2 = np.stack([o.make_weights(rng, qt2, hid, inner) for _ in range(e)])
            w13d, w2d = _dev(w13), _dev(w2)
            ids, wts = _routing(rng, t, e - 1, top_k)            # the last expert has no pairs
            pairs = t * top_k
            # blocks of 16 slots where both formats have such tiles, else of 32
            assert _lib_takes(ops, qtype, qt2, hid, inner, hid, top_k, t, e) == (2 if qtype in (o.Q4_0, o.Q8_0, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS) else 3)
            x = torch.randn(t, hid, device="cuda")
            x = (x * (4.0 / ops.ggml_moe_a8_vec(x, w13d, _dev(ids), top_k, qtype, 2 * inner, t).abs().max())).to(TORCH_DT[dt])
            h = ops.ggml_moe_a8_vec(x, w13d, _dev(ids), top_k, qtype, 2 * inner, t)
            y = ops.ggml_moe_a8_vec(h, w2d, _dev(ids.reshape(pairs, 1)), 1, qt2, hid, pairs, activation="silu")
            want = torch.empty((t, hid), dtype=x.dtype, device="cuda")
            ops.moe_weighted_sum(y.reshape(t, top_k, hid), _dev(wts), want)
            got = ops.moe_vec_layer(x, w13d, w2d, _dev(wts), _dev(ids), qtype, qt2, "silu")
            assert not torch.isnan(want).any()
            # (as for the two-launch route: bit for bit in most cases, a quant of h may move by a step in rare ones)
            err = o.rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy())
            assert err <= {"f32": 5e-4, "f16": 1e-3, "bf16": 4e-3}[dt], f"{o.TYPE_NAMES[qtype]} {o.TYPE_NAMES[qt2]} {dt} case {case} rel-L2 {err}"


TILE16_TYPES = [o.Q4_0, o.Q8_0, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS]


@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("qtype", MMQ_TYPES)
def test_moe_layer_on_grouped_tiles_matches_the_separate_steps(qtype, dt):
    """moe_mmq_layer (the four launches of the tile route with the grouped operator's arithmetic) against
    moe_align_block_size, ggml_moe_a8 twice (the second with the activation) and moe_weighted_sum on the same block
    size: blocks of 16 slots where the experts see few pairs and the format has such tiles, else the reference's blocks
    of 32; from 64 pairs per expert on, layers with a 16-deep format run in slot order on the dense engine with blocks of 64 (cases 4, 5).  More than 64 tokens, inner sizes that end inside a tile of features, an expert without pairs, a second
    format, and a pair whose expert id names no expert (it adds nothing in both)."""
    ops = _ops()
    from vllm_gguf_plugin_prism_amd import _lib, dispatch
    rng = np.random.default_rng(2100 + qtype)
    qk = o.QUANT_SIZES[qtype][0]
    other = o.Q8_0 if qtype != o.Q8_0 else o.Q4_0
    cases = [(70, 2, 12, 512, 768, 16), (24, 4, 8, 256, 1280 if qk == 32 else 1024, 16),
             (70, 4, 8, 512, 768, 32), (40, 2, 3, 256, 1312 if qk == 32 else 1280, 32),
             (300, 2, 5, 512, 768, 128), (300, 1, 3, 256, 1312 if qk == 32 else 1280, 128)]
    for case, (t, top_k, e, hid, inner, block) in enumerate(cases):
        if block == 16 and qtype not in TILE16_TYPES:
            continue
        for qt2 in (qtype, other) if case in (0, 2, 4) else (qtype,):
            w13 = np.stack([o.make_weights(rng, qtype, 2 * inner, hid) for _ in range(e)])
            w2 = np.stack([o.make_weights(rng, qt2, hid, inner) for _ in range(e)])
            w13d, w2d = _dev(w13), _dev(w2)
            ids, wts = _routing(rng, t, e - 1, top_k)            # the last expert has no pairs
            if case % 2 == 1:
                ids[5, top_k - 1] = e + 3
            pairs = t * top_k
            route = _lib.lib().gguf_moe_mmq_layer_takes(int(qtype), int(qt2), hid, inner, hid, top_k, t, e)
            deep16 = bool({int(qtype), int(qt2)} & {o.Q2_K, o.Q3_K, o.Q6_K})   # the dense engine takes layers with a 16-deep format
            assert route == {16: 1, 32: 2, 128: 3 if deep16 else 2}[block], (case, route)
            # (the route in slot order is compared with the operators on the reference's blocks of 32)
            sort_block = min(block, 32)
            sorted_ids, expert_ids, post = ops.moe_align_block_size(_dev(ids), sort_block, e)

            def separate(x):
                h = ops.ggml_moe_a8(x, w13d, sorted_ids, expert_ids, post, qtype, 2 * inner, top_k, t, block_size=sort_block)
                y = ops.ggml_moe_a8(h, w2d, sorted_ids, expert_ids, post, qt2, hid, 1, pairs, activation="silu", block_size=sort_block)
                want = torch.empty((t, hid), dtype=x.dtype, device="cuda")
                ops.moe_weighted_sum(y.reshape(t, top_k, hid), _dev(wts), want)
                return h, want

            x = torch.randn(t, hid, device="cuda")
            x = (x * (4.0 / separate(x)[0].abs().max())).to(TORCH_DT[dt])
            want = separate(x)[1]
            got = ops.moe_mmq_layer(x, w13d, w2d, _dev(wts), _dev(ids), qtype, qt2, "silu")
            assert not torch.isnan(want).any()
            # (bit for bit in most cases; a quant of h may move by a step where the compiler contracts a multiply-add
            #  differently in the two kernels)
            err = o.rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy())
            assert err <= {"f32": 5e-4, "f16": 1e-3, "bf16": 4e-3}[dt], f"{o.TYPE_NAMES[qtype]} {o.TYPE_NAMES[qt2]} {dt} case {case} rel-L2 {err}"
            if dispatch.select_moe_path(int(qtype), int(qt2), t) == "grouped":   # the layer through the dispatcher takes the same call
                assert torch.equal(dispatch.fused_moe_gguf(x, w13d, w2d, _dev(wts), _dev(ids), qtype, qt2, "silu"), got)
            if dt == "f16" and qt2 == qtype and case in (0, 2, 4):   # the other activation the reference's MoE models use
                h = ops.ggml_moe_a8(x, w13d, sorted_ids, expert_ids, post, qtype, 2 * inner, top_k, t, block_size=sort_block)
                y = ops.ggml_moe_a8(h, w2d, sorted_ids, expert_ids, post, qt2, hid, 1, pairs, activation="gelu", block_size=sort_block)
                want_g = torch.empty((t, hid), dtype=x.dtype, device="cuda")
                ops.moe_weighted_sum(y.reshape(t, top_k, hid), _dev(wts), want_g)
                got_g = ops.moe_mmq_layer(x, w13d, w2d, _dev(wts), _dev(ids), qtype, qt2, "gelu")
                assert o.rel_l2(got_g.float().cpu().numpy(), want_g.float().cpu().numpy()) <= 1e-3
    with pytest.raises(ValueError):     # more experts than the tile kernels' guard on expert ids admits
        row = 256 // qk * o.QUANT_SIZES[qtype][1]
        ops.moe_mmq_layer(torch.zeros(70, 256, device="cuda", dtype=TORCH_DT[dt]), _dev(np.zeros((300, 512, row), dtype=np.uint8)),
                          _dev(np.zeros((300, 256, row), dtype=np.uint8)), _dev(np.ones((70, 2), dtype=np.float32)),
                          _dev(np.zeros((70, 2), dtype=np.int32)), qtype, qtype, "silu")


def test_moe_layers_of_a_wide_model_match_the_separate_steps():
    """A layer the size of an 8-expert top-2 model's (hidden 4096, inner 14336, Q4_K gate / up and Q6_K down projections:
    224 tiles of features per block, a second format of another group size): the layer entry points against the
    operators called one by one, below 64 tokens on 16-slot blocks, above on 16 and on 32."""
    ops = _ops()
    from vllm_gguf_plugin_prism_amd import _lib, dispatch, synth
    rng = np.random.default_rng(77)
    e, hid, inner, top_k, qt1, qt2 = 8, 4096, 14336, 2, o.Q4_K, o.Q6_K
    w13d = _dev(np.stack([synth.random_blocks(rng, qt1, 2 * inner, hid) for _ in range(e)]))
    w2d = _dev(np.stack([synth.random_blocks(rng, qt2, hid, inner, 1e-5, 1e-4) for _ in range(e)]))
    for t, want_route in ((48, "vec 2"), (64, "vec 2"), (96, "mmq 2"), (33, "vec 2")):
        ids, wts = _routing(rng, t, e, top_k)
        pairs = t * top_k
        x = torch.randn(t, hid, device="cuda")
        x = x * (4.0 / ops.ggml_moe_a8_vec(x, w13d, _dev(ids), top_k, qt1, 2 * inner, t).abs().max())   # (random blocks: keep h small)
        L = _lib.lib()
        if t <= 64:
            assert L.gguf_moe_vec_layer_takes(qt1, qt2, hid, inner, hid, top_k, t, e) == 2
            h = ops.ggml_moe_a8_vec(x, w13d, _dev(ids), top_k, qt1, 2 * inner, t)
            y = ops.ggml_moe_a8_vec(h, w2d, _dev(ids.reshape(pairs, 1)), 1, qt2, hid, pairs, activation="silu")
        else:
            assert L.gguf_moe_mmq_layer_takes(qt1, qt2, hid, inner, hid, top_k, t, e) == 2    # 24 pairs per expert: blocks of 32
            s_ids, e_ids, post = ops.moe_align_block_size(_dev(ids), 32, e)
            h = ops.ggml_moe_a8(x, w13d, s_ids, e_ids, post, qt1, 2 * inner, top_k, t)
            y = ops.ggml_moe_a8(h, w2d, s_ids, e_ids, post, qt2, hid, 1, pairs, activation="silu")
        want = torch.empty((t, hid), dtype=x.dtype, device="cuda")
        ops.moe_weighted_sum(y.reshape(t, top_k, hid), _dev(wts), want)
        got = dispatch.fused_moe_gguf(x, w13d, w2d, _dev(wts), _dev(ids), qt1, qt2, "silu")
        assert not torch.isnan(want).any() and not torch.isinf(want).any()
        err = o.rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy())
        assert err <= 5e-4, f"t={t} ({want_route}) rel-L2 {err}"


def _lib_takes(ops, *args):
    from vllm_gguf_plugin_prism_amd import _lib
    return _lib.lib().gguf_moe_vec_layer_takes(*[int(a) for a in args])


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("qtype", MMQ_TYPES)
def test_moe_vec_shared_experts_keep_gemv_semantics(qtype, dt):
    """With two or more pairs per expert the per-pair operator runs on the grouped tile kernel (all tile formats but
    Q5_0).  Its results must stay those of the GEMV: for Q4_K / Q5_K the offset term multiplies the quant sums, not the
    stored block sums the tile operator ggml_moe_a8 uses (the two differ by about 1e-2 on these weights)."""
    ops = _ops()
    rng = np.random.default_rng(970 + qtype)
    t, top_k, e, n, k = 40, 4, 8, 200, 768
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    xd, xv = _x(rng, t, k, dt)
    ids, _ = _routing(rng, t, e, top_k)
    y = ops.ggml_moe_a8_vec(xd, _dev(w), _dev(ids), top_k, qtype, n, t)
    assert y.shape == (t * top_k, n) and y.dtype == TORCH_DT[dt]
    want = o.moe_a8_vec(xv, w, ids, top_k, qtype, n, t)
    assert o.rel_l2(y.float().cpu().numpy(), want) <= (1e-5 if dt == "f32" else 1e-3)
    # an expert id outside [0, experts) names no weights: its pairs are left out, the others are unaffected
    bad = ids.copy()
    bad[3, 1] = e + 5
    y2 = ops.ggml_moe_a8_vec(xd, _dev(w), _dev(bad), top_k, qtype, n, t)
    keep = np.ones(t * top_k, dtype=bool)
    keep[3 * top_k + 1] = False
    assert torch.equal(y2[torch.from_numpy(keep).cuda()], y[torch.from_numpy(keep).cuda()])


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q8_0, o.Q4_K, o.Q5_K, o.IQ4_XS, o.IQ2_XXS, o.Q6_K])
def test_mmq_nine_to_32_rows(qtype, dt):
    """9 to 32 rows of X run on 16-row tiles with K split over the chip (Q6_K up to 16 rows, the large tiles above): both
    sides of the 16- and 32-row edges, an output narrower than a tile and one that is not a multiple of it, a short K
    that cannot be split and a long one that is, and the same call without room for partial tiles."""
    ops = _ops()
    rng = np.random.default_rng(1300 + qtype)
    from vllm_gguf_plugin_prism_amd import _lib
    lib = _lib.lib()
    for m, n, k in [(9, 72, 512), (16, 200, 1024), (17, 384, 2048), (32, 130, 4096), (33, 130, 1024)]:
        w = o.make_weights(rng, qtype, n, k)
        xd, xv = _x(rng, m, k, dt)
        y = ops.ggml_mul_mat_a8(_dev(w), xd, qtype, n)
        want = o.mul_mat_a8(w, xv, qtype, n, "mmq")
        tol = 1e-5 if dt == "f32" else 1e-3
        assert o.rel_l2(y.float().cpu().numpy(), want) <= tol, (o.TYPE_NAMES[qtype], m, n, k)
        # the minimum workspace: no room for partial tiles, so K is not split; same arithmetic, other summation order
        nbytes = m * lib.gguf_q8_1_row_bytes(k)
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        y2 = torch.empty_like(y)
        rc = lib.gguf_mmq_engine(_dev(w).data_ptr(), xd.data_ptr(), {"f32": 0, "f16": 1, "bf16": 2}[dt], ws.data_ptr(), y2.data_ptr(),
                                 int(qtype), n, k, m, 1, nbytes, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        assert o.rel_l2(y2.float().cpu().numpy(), want) <= tol


@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q5_K, o.Q6_K, o.Q4_0, o.Q8_0])
def test_mmq_up_to_16_rows_from_packed_blocks(qtype, dt):
    """Q4_K, Q5_K, Q6_K with at most 32 rows of X (and Q4_0, Q8_0 with nine to 16) build their MFMA operands straight from the packed blocks, K split over the waves
    of a workgroup: one super-block of K, a stretch that fills LDS (K = 4096), K beyond it (split over workgroups as
    well, and the same call without room for partial tiles), few columns (split down to a super-block per wave), the
    two-column-tile variant of wide outputs with a ragged last tile, a row slice of a wider weight tensor with bias
    into a column slice of a wider result, and a slice whose rows are not 16-byte aligned (Q4_K / Q5_K take the staged
    kernel there, Q6_K blocks are at even addresses anyway)."""
    ops = _ops()
    rng = np.random.default_rng(1400 + qtype)
    from vllm_gguf_plugin_prism_amd import _lib
    lib = _lib.lib()
    tol = 1e-5 if dt == "f32" else (1e-3 if dt == "f16" else 8e-3)
    for m, n, k in [(9, 72, 256), (16, 200, 4096), (16, 40, 8192), (13, 96, 4096), (12, 10250, 512), (1, 33, 768)]:
        w = o.make_weights(rng, qtype, n, k)
        xd, xv = _x(rng, m, k, dt)
        want = o.mul_mat_a8(w, xv, qtype, n, "mmq")
        if m > 8:
            y = ops.ggml_mul_mat_a8(_dev(w), xd, qtype, n)
            assert o.rel_l2(y.float().cpu().numpy(), want) <= tol, (m, n, k)
        # through the engine entry point with the integer engine named (no GEMV route for few rows) and the minimum
        # workspace
        nbytes = m * lib.gguf_q8_1_row_bytes(k)
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        y2 = torch.empty((m, n), dtype=TORCH_DT[dt], device="cuda")
        rc = lib.gguf_mmq_engine(_dev(w).data_ptr(), xd.data_ptr(), {"f32": 0, "f16": 1, "bf16": 2}[dt], ws.data_ptr(), y2.data_ptr(),
                                 int(qtype), n, k, m, 1, nbytes, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        assert o.rel_l2(y2.float().cpu().numpy(), want) <= tol, (m, n, k, "minimum workspace")
    if qtype in (o.Q4_K, o.Q5_K, o.Q6_K):
        # 17 .. 32 rows: two 16-row tiles of X against every weight operand; 32 and 64 columns per workgroup for wide
        # outputs (ragged last tiles), K beyond 4096 (split over workgroups too)
        for m, n, k in [(17, 72, 256), (32, 200, 4096), (20, 4200, 512), (31, 8300, 256), (24, 40, 8192)]:
            w = o.make_weights(rng, qtype, n, k)
            xd, xv = _x(rng, m, k, dt)
            y = ops.ggml_mul_mat_a8(_dev(w), xd, qtype, n)
            assert o.rel_l2(y.float().cpu().numpy(), o.mul_mat_a8(w, xv, qtype, n, "mmq")) <= tol, (m, n, k)
    # shard of a merged layer: rows 8 .. 8 + n of a taller tensor whose rows are 32 bytes longer than the blocks,
    # bias, result columns 5 .. 5 + n of a wider tensor
    m, n, k = (14 if qtype in (o.Q4_0, o.Q8_0) else 27), 150, 1024
    row_bytes = k // o.QUANT_SIZES[qtype][0] * o.QUANT_SIZES[qtype][1]
    for pad, where in ((32, "aligned"), (2, "unaligned")):
        tall = rng.integers(0, 256, (n + 20, row_bytes + pad), dtype=np.uint8)
        w = o.make_weights(rng, qtype, n, k)
        tall[8:8 + n, :row_bytes] = w
        xd, xv = _x(rng, m, k, dt)
        bias = torch.from_numpy(rng.standard_normal(n).astype(np.float32)).to(TORCH_DT[dt]).cuda()
        wide = torch.full((m, n + 11), 7.0, dtype=TORCH_DT[dt], device="cuda")
        ops.ggml_mul_mat_a8(_dev(tall)[8:8 + n, :row_bytes], xd, qtype, n, out=wide[:, 5:5 + n], bias=bias)
        want = o.mul_mat_a8(w, xv, qtype, n, "mmq") + bias.float().cpu().numpy()
        assert o.rel_l2(wide[:, 5:5 + n].float().cpu().numpy(), want) <= tol, where
        assert torch.all(wide[:, :5] == 7.0) and torch.all(wide[:, 5 + n:] == 7.0)


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q8_0, o.Q4_K, o.Q5_K, o.IQ4_XS, o.IQ2_XXS])
def test_moe_vec_blocks_of_16_slots(qtype, dt):
    """Up to 16 pairs per expert on average the tile route sorts into blocks of 16 slots and runs the 16-row MFMA kernel:
    experts with more than 16 pairs (two blocks), with none, a ragged last step of K (for the 32-value formats), an
    output narrower and one wider than the kernel's 128 features, and an expert id outside the table."""
    ops = _ops()
    rng = np.random.default_rng(1200 + qtype)
    qk = o.QUANT_SIZES[qtype][0]
    for t, top_k, e, n, k in [(24, 4, 8, 200, 736 if qk == 32 else 768), (64, 8, 64, 72, 512)]:
        w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
        xd, xv = _x(rng, t, k, dt)
        ids, _ = _routing(rng, t, e, top_k)
        if e == 8:
            ids[:20, 0] = 5          # expert 5 gets at least 20 pairs: two blocks
            ids[ids == 2] = 3        # expert 2 gets none (pairs are independent: a token may name an expert twice)
        assert 2 * e <= t * top_k <= 16 * e
        y = ops.ggml_moe_a8_vec(xd, _dev(w), _dev(ids), top_k, qtype, n, t)
        want = o.moe_a8_vec(xv, w, ids, top_k, qtype, n, t)
        assert o.rel_l2(y.float().cpu().numpy(), want) <= (1e-5 if dt == "f32" else 1e-3), (o.TYPE_NAMES[qtype], t, e)
        bad = ids.copy()
        bad[1, 0] = e + 3
        y2 = ops.ggml_moe_a8_vec(xd, _dev(w), _dev(bad), top_k, qtype, n, t)
        keep = np.ones(t * top_k, dtype=bool)
        keep[top_k] = False
        assert torch.equal(y2[torch.from_numpy(keep).cuda()], y[torch.from_numpy(keep).cuda()])


@pytest.mark.parametrize("qtype", ALL)
def test_moe_vec_matches_oracle(qtype):
    ops = _ops()
    rng = np.random.default_rng(900 + qtype)
    t, top_k, e, n, k = 9, 4, 8, 96, 512
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    xd, xv = _x(rng, t, k, "f32")
    ids, _ = _routing(rng, t, e, top_k)
    y = ops.ggml_moe_a8_vec(xd, _dev(w), _dev(ids), top_k, qtype, n, t)
    assert y.shape == (t * top_k, n)
    assert o.rel_l2(y.cpu().numpy(), o.moe_a8_vec(xv, w, ids, top_k, qtype, n, t)) <= 1e-5


def test_moe_sum_and_block_size():
    ops = _ops()
    x = torch.randn(5, 4, 32, device="cuda")
    out = torch.empty(5, 32, device="cuda")
    ops.moe_sum(x, out)
    assert torch.allclose(out, x.sum(dim=1))
    assert ops.ggml_moe_get_block_size(2) == ops.ggml_moe_get_block_size(14) > 0
    assert ops.ggml_moe_get_block_size(99) == 0
