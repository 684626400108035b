"""A layer norm with no pass of its own: ``LN(x) . W + b = r (x . W') - r mu colsum(W') + b'``.

The reference runs ``layernorm!`` (layernorm.jl:44-135) and ``matmul!`` (matmul.jl:78-79) as two ops, and the oracle
follows it: normalise in fp32, round the row to fp16, multiply.  The folded form never forms the normalised row (the
fp16 rounding sits on ``gamma W`` instead), so it is held to the parity gate against ``layernorm_f16 -> gemm_f16`` --
max relative error <= 1e-2, cosine >= 0.9999 -- not to the oracle's bits.  The row statistics it needs are checked on
their own against numpy in float64."""
import numpy as np
import pytest

import oracle
from util import assert_parity, poison, to_dev, to_host

pytestmark = pytest.mark.gpu


def _seg_stats(x):
    """(sum, squares about the segment's own mean) of every 32-column segment of every row, float64."""
    x = x.astype(np.float64)
    T, Cn = x.shape
    nseg = (Cn + 31) // 32
    out = np.zeros((T, nseg, 2))
    for s in range(nseg):
        blk = x[:, 32 * s:min(Cn, 32 * s + 32)]
        out[:, s, 0] = blk.sum(1)
        out[:, s, 1] = ((blk - blk.mean(1, keepdims=True)) ** 2).sum(1)
    return out


def _row_moments(stats, Cn):
    """What a consumer makes of the statistics: the row's mean and variance (float64)."""
    nseg = stats.shape[1]
    cnt = np.array([min(32, Cn - 32 * s) for s in range(nseg)], dtype=np.float64)
    mu = stats[:, :, 0].sum(1) / Cn
    m2 = (stats[:, :, 1] + cnt * (stats[:, :, 0] / cnt - mu[:, None]) ** 2).sum(1)
    return mu, m2 / Cn


@pytest.mark.parametrize("T,Cn,mean", [(300, 384, 0.0), (70, 1280, 3.0), (33, 1000, -20.0), (5, 8, 1.0), (129, 5120, 0.5)])
def test_row_statistics(ctx, T, Cn, mean):
    import torch
    import juliavision_amd as jv
    x = oracle.randn_f16((T, Cn), 11, mean, 1.0)
    stats = poison(jv.rowstats_new(T, Cn))
    jv.rowstats_(ctx, stats, to_dev(x))
    torch.cuda.synchronize()
    got, want = to_host(stats).astype(np.float64).transpose(1, 0, 2), _seg_stats(x)      # stored segment-major
    assert np.allclose(got[:, :, 0], want[:, :, 0], rtol=1e-5, atol=1e-4)
    assert np.allclose(got[:, :, 1], want[:, :, 1], rtol=1e-4, atol=1e-4)
    mu, var = _row_moments(got, Cn)
    x64 = x.astype(np.float64)
    assert np.allclose(mu, x64.mean(1), rtol=1e-5, atol=1e-5) and np.allclose(var, x64.var(1), rtol=1e-4)


@pytest.mark.parametrize("K,F,layout,affine", [
    (1280, 5120, "kf", True), (1280, 3840, "fk", True), (384, 1152, "kf", False), (512, 264, "fk", True),
    (300, 1000, "kf", True),          # 16-byte rows, K not a multiple of the k-groups
    (129, 70, "kf", True), (129, 70, "fk", True),     # no 16-byte rows: an element at a time
])
def test_prepared_constants(ctx, K, F, layout, affine):
    """``lnfold_prepare``'s three results against numpy: ``Wp`` = fp16(gamma W) exactly (one rounding of the fp32 product),
    ``colsum`` the column sums of the ROUNDED ``Wp`` and ``biasp`` = b + beta . W to fp32 summation error, in W's layout."""
    import torch
    import juliavision_amd as jv
    W = oracle.randn_f16((K, F), 41, 0, 1.0 / np.sqrt(K))
    g = oracle.randn_f16((K,), 42, 1.0, 0.2) if affine else None
    be = oracle.randn_f16((K,), 43, 0, 0.3) if affine else None
    b = oracle.randn_f16((F,), 44, 0, 0.1)
    Wd = to_dev(W) if layout == "kf" else to_dev(np.ascontiguousarray(W.T)).t()
    fw = jv.lnfold_prepare(ctx, Wd, None if g is None else to_dev(g), None if be is None else to_dev(be), to_dev(b))
    torch.cuda.synchronize()
    assert fw.wp.stride() == Wd.stride()
    wp_want = (W.astype(np.float32) * (g.astype(np.float32)[:, None] if affine else np.float32(1))).astype(np.float16)
    wp_got = fw.wp.cpu().numpy()
    assert np.array_equal(wp_got, wp_want)
    cs_want = wp_want.astype(np.float64).sum(0)
    bp_want = b.astype(np.float64) + ((be.astype(np.float64)[:, None] * W.astype(np.float64)).sum(0) if affine else 0.0)
    assert np.allclose(to_host(fw.colsum), cs_want, rtol=1e-5, atol=1e-5 * np.sqrt(K))
    assert np.allclose(to_host(fw.biasp), bp_want, rtol=1e-5, atol=1e-5 * np.sqrt(K))


def _folded(ctx, T, K, F, *, layout="kf", planes=1, epi="none", residual=False, mean=0.0, out_f32=False, gamma=True, beta=True, seed=21):
    import torch
    import juliavision_amd as jv
    X = oracle.randn_f16((T, K), seed, mean, 1.0)
    W = oracle.randn_f16((K, F), seed + 1, 0, 1.0 / np.sqrt(K))
    b = oracle.randn_f16((F,), seed + 2, 0, 0.1)
    g = oracle.randn_f16((K,), seed + 3, 1.0, 0.2) if gamma else None
    be = oracle.randn_f16((K,), seed + 4, 0.0, 0.2) if beta else None
    R = oracle.randn_f16((T, F), seed + 5) if residual else None
    h, _, _ = oracle.layernorm_f16(X, g, be, 1e-5)
    want = oracle.gemm_f16(h, W, b, epi=epi, residual=R, out_f32=out_f32)
    Wd = to_dev(W) if layout == "kf" else to_dev(np.ascontiguousarray(W.T)).t()
    fw = jv.lnfold_prepare(ctx, Wd, None if g is None else to_dev(g), None if be is None else to_dev(be), to_dev(b), planes=planes)
    dX = to_dev(X)
    stats = jv.rowstats_(ctx, jv.rowstats_new(T, K), dX)
    out = poison(torch.empty((T, F), dtype=torch.float32 if out_f32 else torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.lnfold_matmul_(ctx, out, fw, dX, stats, 1e-5, epi=epi, residual=None if R is None else to_dev(R))
    torch.cuda.synchronize()
    return assert_parity(to_host(out), want, what=f"folded norm T{T} K{K} F{F} {layout} x{planes} {epi}")


@pytest.mark.parametrize("layout", ["kf", "fk"])
@pytest.mark.parametrize("T,K,F,planes", [
    (300, 384, 1152, 1), (300, 384, 1152, 3), (1370, 384, 1536, 1), (1500, 1280, 1280, 1), (1500, 1280, 3840, 3),
    (70, 128, 64, 1), (200, 512, 264, 1), (9, 256, 136, 1),
])
def test_folded_norm_meets_the_two_ops(ctx, T, K, F, planes, layout):
    _folded(ctx, T, K, F, layout=layout, planes=planes)


def test_folded_norm_with_everything_around_it(ctx):
    _folded(ctx, 1500, 1280, 5120, epi="gelu")                    # config 2's first MLP linear behind its norm
    _folded(ctx, 333, 384, 384, residual=True, epi="relu")
    _folded(ctx, 260, 256, 520, out_f32=True)
    _folded(ctx, 260, 256, 520, gamma=False, beta=False)
    _folded(ctx, 260, 256, 520, gamma=True, beta=False, epi="gelu_tanh")
    # rows whose mean is far from zero against their spread: the correction term is most of the accumulator
    _folded(ctx, 400, 1280, 640, mean=8.0)
    _folded(ctx, 400, 384, 1152, mean=-30.0, planes=3)


@pytest.mark.parametrize("T,K,F", [(1500, 5120, 1280), (1370, 384, 384), (1370, 1536, 384), (1500, 1280, 1280), (300, 256, 1024), (4096, 512, 256)])
def test_a_gemm_leaves_the_statistics_of_its_rows(ctx, T, K, F):
    """The producer side, over the tiles and K-split forms the planner picks (the in-launch exchange at 1500 x 5120 ->
    1280, 64 x 64 and 64 x 128 tiles, the four-wave kernel's tiles): Y carries mi_gemm_f16's bits, the statistics are those of the
    final rows -- after the residual -- and a folded norm + linear that consumes them meets the two ops."""
    import torch
    import juliavision_amd as jv
    X = oracle.randn_f16((T, K), 31, 0, 1.0 / np.sqrt(K))
    W, b, R = oracle.randn_f16((K, F), 32), oracle.randn_f16((F,), 33, 0, 0.1), oracle.randn_f16((T, F), 34, 0.3, 1.0)
    dX, dW, db, dR = to_dev(X), to_dev(W), to_dev(b), to_dev(R)
    y0 = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.matmul_(ctx, y0, dW, dX, db, residual=dR)
    y = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
    stats = poison(jv.rowstats_new(T, F))
    ctx.ws.reset()
    jv.matmul_rowstats_(ctx, y, stats, dW, dX, db, residual=dR)
    torch.cuda.synchronize()
    assert_parity(to_host(y), oracle.gemm_f16(X, W, b, residual=R), what="gemm with statistics")
    got, want = to_host(stats).astype(np.float64).transpose(1, 0, 2), _seg_stats(to_host(y))
    assert np.isfinite(got).all()
    assert np.allclose(got[:, :, 0], want[:, :, 0], rtol=1e-5, atol=1e-3) and np.allclose(got[:, :, 1], want[:, :, 1], rtol=1e-4, atol=1e-3)
    # ... and the next linear reads them
    F2 = 512
    W2, g, be = oracle.randn_f16((F, F2), 35, 0, 1.0 / np.sqrt(F)), oracle.randn_f16((F,), 36, 1.0, 0.1), oracle.randn_f16((F,), 37, 0, 0.1)
    fw = jv.lnfold_prepare(ctx, to_dev(W2), to_dev(g), to_dev(be), None)
    out = poison(torch.empty((T, F2), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.lnfold_matmul_(ctx, out, fw, y, stats, 1e-6)
    torch.cuda.synchronize()
    h, _, _ = oracle.layernorm_f16(to_host(y), g, be, 1e-6)
    assert_parity(to_host(out), oracle.gemm_f16(h, W2, None), what="folded norm over a GEMM's own statistics")


def test_folded_norm_declines_what_it_does_not_cover(ctx):
    import torch
    import juliavision_amd as jv
    for (T, K, F) in [(300, 72, 128), (4, 256, 256)]:             # K off the pipelined kernels' 64-deep tiles; decode-sized rows
        W = to_dev(oracle.randn_f16((K, F), 41))
        fw = jv.lnfold_prepare(ctx, W, None, None, None)
        x = to_dev(oracle.randn_f16((T, K), 42))
        stats = jv.rowstats_(ctx, jv.rowstats_new(T, K), x)
        out = torch.empty((T, F), dtype=torch.float16, device="cuda")
        with pytest.raises(jv.DeclineError):
            jv.lnfold_matmul_(ctx, out, fw, x, stats, 1e-5)
