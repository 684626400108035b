"""GEMM parity on the GPU, through the C ABI, against the CPU oracle (mm2 form,
DNNKernels/src/kernels/extern/matmul.jl:17-27,210-214).  Tolerance: max relative
error <= 1e-2 and cosine >= 0.9999 (the gate BASELINE names); the reference's own
tool gate is rel < 2e-2 on 64 rows (tools/gemm_bench.jl:134-157)."""
import numpy as np
import pytest

import oracle
from util import assert_parity, poison, to_dev, to_host

pytestmark = pytest.mark.gpu


def _run(ctx, T, K, F, *, layout="kf", bias=True, epi="none", out_f32=False, residual=False, bias_mode="col", seed=1):
    import torch
    import juliavision_amd as jv
    X = oracle.randn_f16((T, K), seed, 0, 1.0 / np.sqrt(K))
    Wkf = oracle.randn_f16((K, F), seed + 1, 0, 1.0)
    b = oracle.randn_f16((F if bias_mode == "col" else T,), seed + 2, 0, 0.02) if bias else None
    R = oracle.randn_f16((T, F), seed + 3, 0, 1.0) if residual else None
    want = oracle.gemm_f16(X, Wkf, b, w_layout="kf", bias_mode=bias_mode if bias else None, epi=epi, out_f32=out_f32, residual=R)
    Wd = to_dev(Wkf) if layout == "kf" else to_dev(np.ascontiguousarray(Wkf.T)).t()
    out = poison(torch.empty((T, F), dtype=torch.float32 if out_f32 else torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.matmul_(ctx, out, Wd, to_dev(X), None if b is None else to_dev(b), epi=epi,
               residual=None if R is None else to_dev(R), bias_mode=bias_mode if bias else None)
    torch.cuda.synchronize()
    return assert_parity(to_host(out), want, what=f"gemm T{T} K{K} F{F} {layout} {epi}")


@pytest.mark.parametrize("layout", ["kf", "fk"])
@pytest.mark.parametrize("T,K,F", [
    (64, 64, 64), (128, 128, 256), (100, 72, 200), (257, 136, 520), (1, 1280, 1280), (4, 1280, 5120),
    (8, 5120, 1280), (9, 256, 264), (33, 8, 8), (300, 384, 1152), (130, 1536, 384),
])
def test_gemm_shapes(ctx, T, K, F, layout):
    _run(ctx, T, K, F, layout=layout)


@pytest.mark.parametrize("epi", ["none", "gelu", "gelu_tanh", "relu"])
@pytest.mark.parametrize("out_f32", [False, True])
def test_gemm_epilogues(ctx, epi, out_f32):
    _run(ctx, 200, 256, 328, epi=epi, out_f32=out_f32)


def test_gemm_no_bias_row_bias_residual(ctx):
    _run(ctx, 150, 128, 136, bias=False)
    _run(ctx, 150, 128, 136, bias_mode="row")
    _run(ctx, 150, 128, 136, residual=True, epi="gelu")
    _run(ctx, 4, 128, 136, residual=True, epi="gelu")


@pytest.mark.parametrize("layout", ["kf", "fk"])
@pytest.mark.parametrize("T,K,F", [
    (1, 8, 8), (2, 72, 136), (3, 264, 200), (5, 1288, 392), (6, 4104, 128), (7, 640, 1032), (8, 2048, 136),
    (2, 264, 12344), (8, 1544, 9000),
])
def test_decode_sized_rows_ragged_extents(ctx, T, K, F, layout):
    """T <= 8 takes the bandwidth kernels: K not a multiple of their 32- and 512-deep strides, F not a multiple of
    their 128-column blocks, every row count their templates round up from; outputs so wide that a wave of the
    [F][K] kernel walks several columns (more than 8 workgroups of four columns per CU), some waves one more than others."""
    import juliavision_amd as jv
    import torch
    W = torch.zeros((K, F), dtype=torch.float16, device="cuda")
    W = W if layout == "kf" else torch.zeros((F, K), dtype=torch.float16, device="cuda").t()
    plan = jv.mmplan(ctx.dev, torch.zeros((T, F), dtype=torch.float16, device="cuda"), W, torch.zeros((T, K), dtype=torch.float16, device="cuda"))
    assert type(plan).__name__ == "MMSkinnyPlan"
    _run(ctx, T, K, F, layout=layout, seed=40 + T)
    _run(ctx, T, K, F, layout=layout, epi="gelu", residual=True, seed=50 + T)
    _run(ctx, T, K, F, layout=layout, bias=False, out_f32=True, seed=60 + T)
    _run(ctx, T, K, F, layout=layout, bias_mode="row", epi="relu", seed=70 + T)


def test_gemm_unaligned_takes_scalar_path(ctx):
    import juliavision_amd as jv
    import torch
    A = torch.zeros((37, 50), dtype=torch.float16, device="cuda")
    B = torch.zeros((21, 37), dtype=torch.float16, device="cuda")
    out = torch.zeros((21, 50), dtype=torch.float16, device="cuda")
    assert type(jv.mmplan(ctx.dev, out, A, B)).__name__ == "MMScalarPlan"
    _run(ctx, 21, 37, 50)
    _run(ctx, 21, 37, 50, layout="fk", epi="relu")


def test_gemm_config1_full(ctx):
    """BASELINE config 1 at full size against the oracle on every one of the 1500 x 5120 outputs (the reference's own
    device-vs-host check samples 64 rows, tools/gemm_bench.jl:136; the whole product is 5 s of CPU)."""
    import torch
    import juliavision_amd as jv
    T, K, F = 1500, 1280, 5120
    X = oracle.randn_f16((T, K), 11, 0, 1.0 / np.sqrt(K))
    W = oracle.randn_f16((K, F), 12, 0, 1.0 / np.sqrt(K))
    b = oracle.randn_f16((F,), 13, 0, 0.02)
    out = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.matmul_(ctx, out, to_dev(W), to_dev(X), to_dev(b), epi="gelu")
    torch.cuda.synchronize()
    got = to_host(out)
    assert np.all(np.isfinite(got))
    want = oracle.gemm_f16(X, W, b, epi="gelu")
    assert_parity(got, want, what="config1, all rows")
    for rows in (np.r_[0:32], np.r_[1468:1500]):          # and band by band: the first tile and the ragged last one
        assert_parity(got[rows], want[rows], what=f"config1 rows {rows[0]}..{rows[-1]}")
    # linearity in X (size-independent property): f(2x) - bias == 2 (f(x) - bias) without epilogue
    o1 = torch.empty((T, F), dtype=torch.float32, device="cuda")
    o2 = torch.empty((T, F), dtype=torch.float32, device="cuda")
    jv.matmul_(ctx, o1, to_dev(W), to_dev(X))
    jv.matmul_(ctx, o2, to_dev(W), to_dev((X.astype(np.float32) * 2).astype(np.float16)))
    torch.cuda.synchronize()
    assert torch.allclose(o2, 2 * o1, rtol=1e-5, atol=1e-5)


def test_batched(ctx):
    import torch
    import juliavision_amd as jv
    # the reference's bmm shapes are (64,1370,6) K=1370 and (1370,1370,6) K=64 (test_batchedmatmul.jl:76-77); scaled down
    for (nb, T, K, F) in [(6, 137, 64, 136), (3, 70, 136, 64), (2, 40, 37, 50)]:
        X = oracle.randn_f16((nb, T, K), 21, 0, 1.0 / np.sqrt(K))
        W = oracle.randn_f16((nb, K, F), 22)
        want = oracle.gemm_f16(X, W)
        out = poison(torch.empty((nb, T, F), dtype=torch.float16, device="cuda"))
        jv.batchedmatmul_(ctx, out, to_dev(W), to_dev(X))
        torch.cuda.synchronize()
        assert_parity(to_host(out), want, what=f"bmm {nb} {T} {K} {F}")


def test_batched_shared_activations_with_per_plane_bias(ctx):
    """q, k, v projections as one launch through the C ABI: X shared (plane stride 0), W, bias and Y per plane."""
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    T, K, F = 300, 256, 384
    X = oracle.randn_f16((T, K), 31, 0, 1.0 / np.sqrt(K))
    W = oracle.randn_f16((3, K, F), 32)
    b = oracle.randn_f16((3, F), 33, 0, 0.5)
    dX, dW, db = to_dev(X), to_dev(W), to_dev(b)
    out = poison(torch.empty((3, T, F), dtype=torch.float16, device="cuda"))
    rc = lib.mi_gemm_f16_batched(out.data_ptr(), dX.data_ptr(), dW.data_ptr(), db.data_ptr(), None, T, K, F, F, K, F,
                                 L.W_KF, L.BIAS_COL, L.EPI["none"], L.F16, 3, T * F, 0, K * F, F, None, 0,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    got = to_host(out)
    for i in range(3):
        assert_parity(got[i], oracle.gemm_f16(X, W[i], b[i]), what=f"qkv plane {i}")


@pytest.mark.parametrize("layout", ["kf", "fk"])
def test_tile_shapes_between_the_big_and_the_small_tile(ctx, layout):
    """The tile is chosen from the grid it gives: 192 x 128 where 128 x 256 tiles would cover half to three quarters
    of the CUs (ragged last row and column tiles), 64 x 128 on mid-sized outputs, 64 x 64 on few tiles and on
    outputs of at most 64 columns."""
    _run(ctx, 1500, 128, 3000, layout=layout, epi="gelu", residual=True, seed=31)      # 144 big tiles -> 8 x 24 of 192 x 128
    _run(ctx, 1500, 192, 1288, layout=layout, residual=True, seed=32)                  # 132 tiles of 128 x 128 -> 24 x 11 of 64 x 128
    _run(ctx, 700, 256, 392, layout=layout, epi="relu", seed=33)                       # 24 tiles -> 11 x 7 of 64 x 64
    _run(ctx, 20000, 128, 64, layout=layout, seed=34)                                  # 64 columns: 64 x 64 tiles, not half-empty 128-wide ones
    _run(ctx, 3000, 128, 40, layout=layout, out_f32=True, seed=35)


@pytest.mark.parametrize("layout", ["kf", "fk"])
def test_split_k_narrow_outputs(ctx, layout):
    """Few output tiles and a deep K: the library splits K over workgroups (fp32 planes in the workspace,
    summed by a second kernel that applies bias, activation and residual)."""
    from juliavision_amd import _lib as L
    lib = L.load()
    assert lib.mi_gemm_f16_workspace(1500, 5120, 1280, L.W_KF, 1) >= 2 * 1500 * 1280 * 4
    ws = lib.mi_gemm_f16_workspace(200, 4096, 256, L.W_KF, 1)
    assert ws >= 2 * 200 * 256 * 4 and ws % (200 * 256 * 4) == 0         # whole fp32 planes of the output
    assert lib.mi_gemm_f16_workspace(200, 128, 256, L.W_KF, 1) == 0      # two 64-deep steps: nothing to split
    assert lib.mi_gemm_f16_workspace(1370, 1536, 384, L.W_KF, 1) == 0    # one pass of 64 x 64 tiles is cheaper than planes
    _run(ctx, 200, 4096, 256, layout=layout, epi="gelu", residual=True)
    _run(ctx, 200, 4096, 256, layout=layout, out_f32=True)
    _run(ctx, 200, 2048, 256, layout=layout, epi="gelu", residual=True)
    _run(ctx, 1500, 5120, 1280, layout=layout, residual=True, seed=7)


def test_split_k_partials_exchanged_inside_the_launch(ctx):
    """Config 2's second MLP linear (1500 x 5120 -> 1280) splits K over two workgroups per 128 x 128 tile that exchange
    their partial tiles through L2 and per-wave arrival flags instead of writing fp32 planes.  The flags carry a
    per-launch epoch and are cleared by their last reader: forty launches back to back on one stream, alternating two
    problems in one workspace, must each give the bits of the first launch of that problem; and the result meets the
    oracle."""
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    st = torch.cuda.current_stream().cuda_stream
    cases = []
    for (T, K, F, seed) in ((1500, 5120, 1280, 3), (700, 2560, 640, 4)):
        X = oracle.randn_f16((T, K), seed, 0, 1.0 / np.sqrt(K))
        W = oracle.randn_f16((K, F), seed + 10)
        b = oracle.randn_f16((F,), seed + 20, 0, 0.02)
        R = oracle.randn_f16((T, F), seed + 30)
        need = lib.mi_gemm_f16_workspace(T, K, F, L.W_KF, 1)
        assert need > 0
        cases.append((T, K, F, X, W, b, R, to_dev(X), to_dev(W), to_dev(b), to_dev(R), need))
    ws = torch.empty(max(c[-1] for c in cases), dtype=torch.uint8, device="cuda")
    outs = [[], []]
    for rep in range(20):
        for ci, (T, K, F, X, W, b, R, dX, dW, db, dR, need) in enumerate(cases):
            y = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
            rc = lib.mi_gemm_f16(y.data_ptr(), dX.data_ptr(), dW.data_ptr(), db.data_ptr(), dR.data_ptr(), T, K, F, F, K, F,
                                 L.W_KF, L.BIAS_COL, L.EPI["gelu"], L.F16, ws.data_ptr(), need, st)
            assert rc == L.OK
            outs[ci].append(y)
    torch.cuda.synchronize()
    for ci, (T, K, F, X, W, b, R, *_rest) in enumerate(cases):
        first = to_host(outs[ci][0])
        assert_parity(first, oracle.gemm_f16(X, W, b, epi="gelu", residual=R), what=f"peer split-K {T}x{K}x{F}")
        for y in outs[ci][1:]:
            assert np.array_equal(to_host(y).view(np.uint16), first.view(np.uint16)), "a later launch differs from the first"


@pytest.mark.parametrize("layout", ["kf", "fk"])
@pytest.mark.parametrize("T,K,F", [(1, 1280, 1280), (4, 1280, 3840), (8, 264, 136), (3, 2048, 520), (1, 1280, 10008)])
def test_layer_norm_folded_into_decode_sized_gemv(ctx, T, K, F, layout):
    """ln_matmul_ against the oracle's layernorm -> gemm, and bit for bit against the two device calls in sequence."""
    import torch
    import juliavision_amd as jv
    X = oracle.randn_f16((T, K), 81, 0.3, 2.0)
    Wkf = oracle.randn_f16((K, F), 82, 0, 1.0 / np.sqrt(K))
    g, be, b = oracle.randn_f16((K,), 83, 1.0, 0.2), oracle.randn_f16((K,), 84, 0, 0.2), oracle.randn_f16((F,), 85, 0, 0.1)
    R = oracle.randn_f16((T, F), 86)
    Wd = to_dev(Wkf) if layout == "kf" else to_dev(np.ascontiguousarray(Wkf.T)).t()
    dX, dg, dbe, db, dR = to_dev(X), to_dev(g), to_dev(be), to_dev(b), to_dev(R)
    for (gamma, beta, hg, hb) in ((dg, dbe, g, be), (None, None, None, None), (dg, None, g, None)):
        h, _, _ = oracle.layernorm_f16(X, hg, hb, 1e-5)
        want = oracle.gemm_f16(h, Wkf, b, epi="gelu", residual=R)
        out = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
        ctx.ws.reset()
        jv.ln_matmul_(ctx, out, Wd, dX, gamma, beta, 1e-5, db, epi="gelu", residual=dR)
        two = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
        hn = torch.empty_like(dX)
        jv.layernorm_(ctx, hn, None, None, dX, gamma, beta, K, 1e-5)
        ctx.ws.reset()
        jv.matmul_(ctx, two, Wd, hn, db, epi="gelu", residual=dR)
        torch.cuda.synchronize()
        assert_parity(to_host(out), want, what=f"ln+gemv T{T} K{K} F{F} {layout}")
        assert np.array_equal(to_host(out), to_host(two)), "folded norm differs from layernorm_ followed by matmul_"
    with pytest.raises(jv.DeclineError):
        jv.ln_matmul_(ctx, torch.empty((16, F), dtype=torch.float16, device="cuda"), Wd, torch.zeros((16, K), dtype=torch.float16, device="cuda"), None, None, 1e-5)


@pytest.mark.parametrize("layout", ["kf", "fk"])
@pytest.mark.parametrize("T,K,F", [(1370, 384, 1152), (1370, 384, 1536), (300, 512, 200), (65, 128, 72), (1000, 256, 3000), (64, 448, 64)])
def test_layer_norm_as_prologue_of_the_tiled_gemm(ctx, T, K, F, layout):
    """ln_matmul_ for T > 8 (the tiled kernel normalises its 64-row panel of X in LDS before the K loop): against the
    oracle's layernorm -> gemm, and bit for bit against layernorm_ followed by matmul_.  Config 3's qkv and fc1
    shapes, ragged last row and column tiles, both tile widths, K at both ends of the supported range."""
    import torch
    import juliavision_amd as jv
    from juliavision_amd.kernels import ln_matmul_folds
    assert ln_matmul_folds(T, K, F)
    X = oracle.randn_f16((T, K), 91, 0.3, 2.0)
    Wkf = oracle.randn_f16((K, F), 92, 0, 1.0 / np.sqrt(K))
    g, be, b = oracle.randn_f16((K,), 93, 1.0, 0.2), oracle.randn_f16((K,), 94, 0, 0.2), oracle.randn_f16((F,), 95, 0, 0.1)
    R = oracle.randn_f16((T, F), 96)
    Wd = to_dev(Wkf) if layout == "kf" else to_dev(np.ascontiguousarray(Wkf.T)).t()
    dX, dg, dbe, db, dR = to_dev(X), to_dev(g), to_dev(be), to_dev(b), to_dev(R)
    for (gamma, beta, hg, hb, epi, res) in ((dg, dbe, g, be, "gelu", True), (None, None, None, None, "none", False), (dg, None, g, None, "relu", True)):
        h, _, _ = oracle.layernorm_f16(X, hg, hb, 1e-6)
        want = oracle.gemm_f16(h, Wkf, b, epi=epi, residual=R if res else None)
        out = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
        ctx.ws.reset()
        jv.ln_matmul_(ctx, out, Wd, dX, gamma, beta, 1e-6, db, epi=epi, residual=dR if res else None)
        two = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
        hn = torch.empty_like(dX)
        jv.layernorm_(ctx, hn, None, None, dX, gamma, beta, K, 1e-6)
        ctx.ws.reset()
        jv.matmul_(ctx, two, Wd, hn, db, epi=epi, residual=dR if res else None)
        torch.cuda.synchronize()
        assert_parity(to_host(out), want, what=f"ln+gemm T{T} K{K} F{F} {layout} {epi}")
        assert np.array_equal(to_host(out), to_host(two)), "norm prologue differs from layernorm_ followed by matmul_"


def test_layer_norm_prologue_declines_what_it_cannot_hold(ctx):
    import torch
    import juliavision_amd as jv
    from juliavision_amd.kernels import ln_matmul_folds
    assert not ln_matmul_folds(1500, 1280, 1280) and not ln_matmul_folds(100, 576, 128) and not ln_matmul_folds(100, 200, 128)
    assert ln_matmul_folds(4, 1280, 1280) and ln_matmul_folds(1370, 384, 1152)
    z = lambda *sh: torch.zeros(sh, dtype=torch.float16, device="cuda")
    for (T, K, F) in ((100, 576, 128), (100, 1280, 128)):
        with pytest.raises(jv.DeclineError):
            jv.ln_matmul_(ctx, z(T, F), z(K, F), z(T, K), None, None, 1e-5)


@pytest.mark.parametrize("layout", ["kf", "fk"])
def test_output_larger_than_2g_elements_is_indexed_in_64_bits(ctx, layout):
    """70 000 x 32 768 outputs (2.29e9 elements, 4.6 GB of fp16): row offsets pass 2^31.  The oracle checks rows at
    the start, around the 2^31-element boundary (row 65 536) and at the end; every row is checked for coverage."""
    import torch
    import juliavision_amd as jv
    T, K, F = 70000, 128, 32768
    Wkf = oracle.randn_f16((K, F), 3, 0, 1.0)
    b = oracle.randn_f16((F,), 4, 0, 0.5)
    rows = np.r_[0:4, 65534:65540, T - 4:T]
    X = torch.empty((T, K), dtype=torch.float16, device="cuda")
    X.normal_(0, 1.0 / np.sqrt(K))
    Xs = oracle.randn_f16((len(rows), K), 5, 0, 1.0 / np.sqrt(K))
    X[torch.from_numpy(rows).cuda()] = to_dev(Xs)
    Wd = to_dev(Wkf) if layout == "kf" else to_dev(np.ascontiguousarray(Wkf.T)).t()
    out = torch.empty((T, F), dtype=torch.float16, device="cuda")
    out.fill_(float("nan"))
    ctx.ws.reset()
    jv.matmul_(ctx, out, Wd, X, to_dev(b), epi="gelu")
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())                         # nothing unwritten anywhere
    want = oracle.gemm_f16(Xs, Wkf, b, epi="gelu")
    assert_parity(to_host(out[torch.from_numpy(rows).cuda()]), want, what=f"rows across the 2^31 boundary, {layout}")
    del out, X
    torch.cuda.empty_cache()


@pytest.mark.parametrize("layout", ["kf", "fk"])
@pytest.mark.parametrize("T,K,F", [(1370, 1536, 384), (200, 2048, 256), (1500, 5120, 1280), (200, 256, 328), (4, 1280, 1280), (77, 2048, 264),
                                   (1370, 384, 384), (64, 128, 64), (130, 512, 1024), (1000, 256, 520), (2500, 128, 192), (65, 1536, 384),
                                   (9, 192, 8), (40, 2048, 376), (8190, 128, 384), (8200, 128, 384), (33, 2112, 384)])
def test_layer_norm_of_the_output_rides_in_the_gemm(ctx, T, K, F, layout):
    """matmul_ln_ against the oracle's gemm -> layernorm, and bit for bit (both outputs) against matmul_ followed by
    layernorm_: split-K shapes (the norm is in the plane-summing pass), unsplit and decode-sized ones (two kernels; one
    to sixteen column tiles a row panel, one and two chunks a lane in the norm, ragged last panels, rows of eight
    columns, eight thousand rows of 384)."""
    import torch
    import juliavision_amd as jv
    X = oracle.randn_f16((T, K), 91, 0, 1.0 / np.sqrt(K))
    Wkf = oracle.randn_f16((K, F), 92, 0, 1.0)
    b, R = oracle.randn_f16((F,), 93, 0, 0.1), oracle.randn_f16((T, F), 94, 0.2, 1.0)
    g, be = oracle.randn_f16((F,), 95, 1.0, 0.2), oracle.randn_f16((F,), 96, 0, 0.2)
    Wd = to_dev(Wkf) if layout == "kf" else to_dev(np.ascontiguousarray(Wkf.T)).t()
    dX, db, dR = to_dev(X), to_dev(b), to_dev(R)
    for (gamma, beta, hg, hb, epi) in ((to_dev(g), to_dev(be), g, be, "none"), (None, None, None, None, "gelu"), (to_dev(g), None, g, None, "relu")):
        y = oracle.gemm_f16(X, Wkf, b, epi=epi, residual=R)
        h, _, _ = oracle.layernorm_f16(y, hg, hb, 1e-6)
        out, normed = (poison(torch.empty((T, F), dtype=torch.float16, device="cuda")) for _ in range(2))
        ctx.ws.reset()
        jv.matmul_ln_(ctx, out, normed, Wd, dX, gamma, beta, 1e-6, db, epi=epi, residual=dR)
        out2, normed2 = (poison(torch.empty((T, F), dtype=torch.float16, device="cuda")) for _ in range(2))
        ctx.ws.reset()
        jv.matmul_(ctx, out2, Wd, dX, db, epi=epi, residual=dR)
        jv.layernorm_(ctx, normed2, None, None, out2, gamma, beta, F, 1e-6)
        torch.cuda.synchronize()
        assert_parity(to_host(out), y, what=f"matmul_ln_ output T{T} K{K} F{F} {layout}")
        assert_parity(to_host(normed), h, what=f"matmul_ln_ norm T{T} K{K} F{F} {layout}")
        assert np.array_equal(to_host(out), to_host(out2)) and np.array_equal(to_host(normed), to_host(normed2))


def test_in_launch_exchanges_on_two_streams_do_not_meet(ctx):
    """Launches that overlap on one GPU take different banks of flag words: the same split-K problem issued alternately
    on two streams, twelve times each without a synchronisation in between, gives the bits of a launch that ran alone."""
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    T, K, F = 1500, 5120, 1280
    x = to_dev(oracle.randn_f16((T, K), 51, 0, 1.0 / np.sqrt(K)))
    w = to_dev(oracle.randn_f16((K, F), 52))
    b, r = to_dev(oracle.randn_f16((F,), 53, 0, 0.02)), to_dev(oracle.randn_f16((T, F), 54))
    need = lib.mi_gemm_f16_workspace(T, K, F, L.W_KF, 1)
    assert need > 0

    def launch(y, ws, stream):
        rc = lib.mi_gemm_f16(y.data_ptr(), x.data_ptr(), w.data_ptr(), b.data_ptr(), r.data_ptr(), T, K, F, F, K, F,
                             L.W_KF, L.BIAS_COL, L.EPI["none"], L.F16, ws.data_ptr(), need, stream.cuda_stream)
        assert rc == L.OK

    alone = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
    ws0 = torch.empty(need, dtype=torch.uint8, device="cuda")
    launch(alone, ws0, torch.cuda.current_stream())
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    wss = [torch.empty(need, dtype=torch.uint8, device="cuda") for _ in streams]      # a workspace belongs to one stream at a time
    outs = [[poison(torch.empty((T, F), dtype=torch.float16, device="cuda")) for _ in range(12)] for _ in streams]
    torch.cuda.synchronize()
    for i in range(12):
        for s, stream in enumerate(streams):
            launch(outs[s][i], wss[s], stream)
    torch.cuda.synchronize()
    for s in range(2):
        for y in outs[s]:
            assert torch.equal(y.view(torch.int16), alone.view(torch.int16))
    assert lib.mi_device_status(0) == 0, "a workgroup gave up waiting for its partner"


def test_a_missed_exchange_is_loud(ctx):
    """A workgroup of the in-launch split-K exchange waits for its partners a bounded time.  The waits are made to fail
    from the host (mi_test_exchange_faults: a handful of polls, and partners that publish an epoch nobody waits for, or
    that seem to sit on another XCD), so every kernel still runs to its end: the call returns MI_OK as always, the
    device's sticky status word names the reason, Y holds NaN instead of a plausible sum, and after the reset that
    mi_device_status(1) performs the same launch is right again.  With the exchange switched off the K-slices go
    through planes."""
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    st = torch.cuda.current_stream().cuda_stream
    T, K, F = 1500, 5120, 1280
    X, W = oracle.randn_f16((T, K), 81, 0, 1.0 / np.sqrt(K)), oracle.randn_f16((K, F), 82)
    b, R = oracle.randn_f16((F,), 83, 0, 0.02), oracle.randn_f16((T, F), 84)
    dX, dW, db, dR = to_dev(X), to_dev(W), to_dev(b), to_dev(R)

    def launch():
        need = lib.mi_gemm_f16_workspace(T, K, F, L.W_KF, 1)
        ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
        y = torch.zeros((T, F), dtype=torch.float16, device="cuda")
        rc = lib.mi_gemm_f16(y.data_ptr(), dX.data_ptr(), dW.data_ptr(), db.data_ptr(), dR.data_ptr(), T, K, F, F, K, F,
                             L.W_KF, L.BIAS_COL, L.EPI["none"], L.F16, ws.data_ptr(), need, st)
        assert rc == L.OK
        torch.cuda.synchronize()
        return y

    assert lib.mi_device_status(1) == 0
    try:
        lib.mi_test_exchange_faults(16, 0x5A5A5, 0)
        y = launch()
        assert lib.mi_device_status(0) == 1, "a wait that gave up must raise MI_DEVSTAT_EXCHANGE_TIMEOUT"
        assert lib.mi_device_status(1) == 1 and lib.mi_device_status(0) == 0      # sticky until reset
        assert bool(torch.isnan(y).all()), "no workgroup may store a sum it could not complete"
        lib.mi_test_exchange_faults(0, 0, 1)
        y = launch()
        assert lib.mi_device_status(1) == 2, "partners on another XCD must raise MI_DEVSTAT_EXCHANGE_XCD"
        assert bool(torch.isnan(y).all())
    finally:
        lib.mi_test_exchange_faults(0, 0, 0)
        lib.mi_device_status(1)
    peer = launch()
    assert lib.mi_device_status(0) == 0
    assert_parity(to_host(peer), oracle.gemm_f16(X, W, b, residual=R), what="exchange after a reset")
    try:
        lib.mi_set_in_launch_exchange(0)
        planes = launch()
    finally:
        lib.mi_set_in_launch_exchange(1)
    assert lib.mi_device_status(0) == 0
    assert_parity(to_host(planes), oracle.gemm_f16(X, W, b, residual=R), what="K-slices through planes")


@pytest.mark.parametrize("T,K,F", [(1500, 5120, 1280), (1370, 1536, 384)])
def test_in_launch_exchange_starts_clean_on_every_replay(ctx, T, K, F):
    """A captured launch carries the flag bank and epoch it was given at capture.  The split-K exchange
    (1500 x 5120 -> 1280) leaves its flags at zero, so a replay waits for this replay's partners and not for what the
    last replay left behind: three replays over changing inputs each equal the eager result on the same inputs, bit
    for bit (the second shape runs without an exchange)."""
    import torch
    import juliavision_amd as jv
    from juliavision_amd.decode import StepGraph
    w = to_dev(oracle.randn_f16((K, F), 61, 0, 1.0))
    b, r = to_dev(oracle.randn_f16((F,), 62, 0, 0.1)), to_dev(oracle.randn_f16((T, F), 63, 0.2, 1.0))
    g, be = to_dev(oracle.randn_f16((F,), 64, 1.0, 0.2)), to_dev(oracle.randn_f16((F,), 65, 0, 0.2))
    x = to_dev(oracle.randn_f16((T, K), 66, 0, 1.0 / np.sqrt(K)))
    y, h = (poison(torch.empty((T, F), dtype=torch.float16, device="cuda")) for _ in range(2))

    def step():
        ctx.ws.reset()
        jv.matmul_ln_(ctx, y, h, w, x, g, be, 1e-6, b, residual=r)

    graph = StepGraph(step)
    for it in range(3):
        x.copy_(to_dev(oracle.randn_f16((T, K), 70 + it, 0, 1.0 / np.sqrt(K))))
        poison(y), poison(h)
        graph.replay()
        torch.cuda.synchronize()
        y2, h2 = (poison(torch.empty_like(y)) for _ in range(2))
        ctx.ws.reset()
        jv.matmul_(ctx, y2, w, x, b, residual=r)
        jv.layernorm_(ctx, h2, None, None, y2, g, be, F, 1e-6)
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), y2.view(torch.int16)) and torch.equal(h.view(torch.int16), h2.view(torch.int16)), it


@pytest.mark.parametrize("T,K,F,with_norm", [(300, 256, 384, True), (200, 2048, 256, True), (130, 128, 520, False), (4, 256, 384, True)])
def test_matmul_with_clamp_in_the_store_is_the_separate_ops(ctx, T, K, F, with_norm):
    """mi_gemm_clamp_ln_f16: GEMM + residual, then aten::clamp, then the layer norm of the clamped rows -- in the
    tiled kernel's store, in the split-K plane sum (K = 2048 over few tiles), and as a pass of its own behind the
    decode-sized kernel (T = 4).  Values are scaled to overflow fp16 in places, so the clamp has something to do."""
    import torch
    import juliavision_amd as jv
    x = to_dev(oracle.randn_f16((T, K), 41, std=30.0))
    w = to_dev(oracle.randn_f16((K, F), 42, std=1200.0 / K ** 0.5))       # sums of std 36 000 whatever K
    b = to_dev(oracle.randn_f16((F,), 43))
    r = to_dev(oracle.randn_f16((T, F), 44, std=1000.0))
    g, be = to_dev(oracle.randn_f16((F,), 45, mean=1.0, std=0.1)), to_dev(oracle.randn_f16((F,), 46, std=0.1))
    y0 = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.matmul_(ctx, y0, w, x, b, residual=r)
    assert bool(torch.isinf(y0).any()) and bool((y0.abs() > 64504).sum() > 100)      # the unclamped result overflows
    want_y = poison(torch.empty_like(y0))
    jv.clamp_(ctx, want_y, y0, -64504.0, 64504.0)
    want_h = poison(torch.empty_like(y0))
    jv.layernorm_(ctx, want_h, None, None, want_y, g, be, F, 1e-5)
    y, h = poison(torch.empty_like(y0)), poison(torch.empty_like(y0))
    ctx.ws.reset()
    jv.matmul_ln_(ctx, y, h if with_norm else None, w, x, g, be, 1e-5, b, residual=r, clamp=64504.0)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y).all()) and torch.equal(y.view(torch.int16), want_y.view(torch.int16))
    if with_norm:
        assert torch.equal(h.view(torch.int16), want_h.view(torch.int16))


def test_clamped_gemm_declines_a_clamp_that_is_not_positive(ctx):
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    x = torch.zeros((16, 64), dtype=torch.float16, device="cuda")
    w = torch.zeros((64, 64), dtype=torch.float16, device="cuda")
    y = torch.zeros((16, 64), dtype=torch.float16, device="cuda")
    for bad in (0.0, -1.0, float("nan")):
        rc = lib.mi_gemm_clamp_ln_f16(y.data_ptr(), None, x.data_ptr(), w.data_ptr(), None, None, None, None, 1e-5, bad,
                                      16, 64, 64, 64, 64, L.W_KF, L.BIAS_NONE, L.EPI["none"], None, 0, ctx.stream)
        assert rc == L.DECLINE_OPERANDS
