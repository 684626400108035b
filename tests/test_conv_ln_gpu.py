"""Convolution-as-GEMM, layer norm and residual add on the GPU through the C ABI,
against the oracle's direct convolution (conv.jl:26-51), two-pass layer norm
(layernorm.jl:53-113) and fp16 add.  Conv shapes include the reference's own test
list (test_convtranspose_gemm.jl:188-191, scaled where large) and BASELINE configs 3/4."""
import numpy as np
import pytest

import oracle
from util import assert_parity, poison, to_dev, to_host

pytestmark = pytest.mark.gpu


def _conv(ctx, N, Cin, H, W, Cout, KH, KW, s, p, d=1, groups=1, bias=True, relu=False, expect=None, seed=1):
    """``s``, ``p``, ``d``: one number for both axes or an ``(x, y)`` pair."""
    import torch
    import juliavision_amd as jv
    pair = lambda v: v if isinstance(v, tuple) else (v, v)
    s, p, d = pair(s), pair(p), pair(d)
    x = oracle.randn_f16((N, Cin, H, W), seed)
    w = oracle.randn_f16((Cout, Cin // groups, KH, KW), seed + 1, 0, 0.05)
    b = oracle.randn_f16((Cout,), seed + 2, 0, 0.5) if bias else None
    want = oracle.conv2d_f16(x, w, b, s[::-1], p[::-1], d[::-1], groups, relu)      # the oracle takes (y, x) pairs as torch does
    out = poison(torch.empty(want.shape, dtype=torch.float16, device="cuda"))
    dx, dw = to_dev(x), to_dev(w)
    plan = jv.conv_plan(ctx.dev, out, dx, dw, s, p, d, groups)
    if expect:
        assert plan.path == expect, plan
    ctx.ws.reset()
    jv.convolution_(ctx, out, dx, dw, None if b is None else to_dev(b), s, p, d, groups, act="relu" if relu else "none")
    torch.cuda.synchronize()
    assert_parity(to_host(out), want, what=f"conv {N},{Cin},{H},{W}->{Cout} k{KH} s{s} p{p} g{groups}")


@pytest.mark.parametrize("N,Cin,H,W,Cout,K,s,p", [
    (1, 3, 64, 64, 144, 7, 4, 3),      # stem shape of test_convtranspose_gemm.jl:188 at 64x64
    (1, 5, 64, 64, 32, 3, 1, 1),
    (1, 7, 48, 48, 48, 5, 2, 2),
    (2, 32, 32, 32, 64, 3, 1, 1),
    (1, 3, 70, 70, 384, 14, 14, 0),    # patch embed 14x14 / stride 14 (config 3) on a 5x5 patch grid
])
def test_conv_im2col(ctx, N, Cin, H, W, Cout, K, s, p):
    _conv(ctx, N, Cin, H, W, Cout, K, K, s, p, expect="im2col_gemm")


@pytest.mark.parametrize("N,Cin,H,W,Cout,KH,KW,s,p,d,kw", [
    (1, 256, 16, 16, 256, 3, 3, 1, 1, 1, {}),                      # config 4's 3x3 256->256 on a small map
    (2, 64, 24, 24, 100, 3, 3, 1, 1, 1, {"relu": True}),           # two images, ragged Cout, relu
    (1, 64, 40, 40, 64, 7, 7, 1, 3, 1, {"bias": False}),           # taps shifted by -3..3 columns: odd and even starts
    (1, 128, 20, 24, 96, 5, 5, 1, (4, 2), (2, 1), {}),             # dilation 2 along x only, unequal padding
    (1, 64, 18, 16, 48, 3, 1, (1, 2), (0, 1), 1, {}),              # 3 rows x 1 column, stride 2 along y, no x padding
    (1, 192, 12, 32, 32, 1, 3, 1, (1, 0), 1, {}),                  # KH = 1, KW = 3
    (3, 64, 9, 10, 40, 3, 3, 1, (0, 2), 1, {"relu": True}),        # OW = 8 without x padding, three images
    (1, 512, 32, 32, 128, 3, 3, 1, 1, 1, {"relu": True}),          # K = 4608 over eight output tiles: split into fp32 planes
])
def test_conv_implicit_gemm(ctx, N, Cin, H, W, Cout, KH, KW, s, p, d, kw):
    _conv(ctx, N, Cin, H, W, Cout, KH, KW, s, p, d, expect="implicit_gemm", **kw)


def test_conv_1x1_and_relu_and_nobias(ctx):
    _conv(ctx, 2, 144, 16, 16, 256, 1, 1, 1, 0, expect="gemm_1x1")
    _conv(ctx, 1, 24, 5, 7, 40, 1, 1, 1, 0, expect="gemm_1x1")          # PQ = 35: scalar GEMM inside
    _conv(ctx, 1, 16, 12, 12, 32, 3, 3, 1, 1, relu=True, bias=False)
    _conv(ctx, 1, 8, 20, 20, 16, 3, 3, 2, 2, d=2)


@pytest.mark.parametrize("N,Cin,H,W,Cout,K,s,p,res,relu", [
    (1, 3, 70, 70, 384, 14, 14, 0, "shared", False),      # a ViT-S/14 patch embedding on a 5 x 5 grid: 588 taps -> 640
    (1, 3, 518, 518, 384, 14, 14, 0, "shared", False),    # config 3's, full size
    (2, 3, 56, 56, 64, 8, 8, 0, "shared", False),         # one position embedding for two images
    (2, 3, 56, 56, 64, 8, 8, 0, "each", True),            # a residual per image, relu before it
    (3, 5, 20, 24, 40, 3, 1, 1, None, False),             # overlapping taps with padding, 45 -> 48 taps
    (1, 16, 9, 9, 24, 4, 4, 0, "shared", False),          # a 2 x 2 grid: four tokens (the decode-sized GEMM inside)
])
def test_conv_writes_tokens_with_the_position_embedding(ctx, N, Cin, H, W, Cout, K, s, p, res, relu):
    """mi_conv2d_tokens_f16 into rows 1.. of a token matrix (row 0 stays as it was), against the oracle's direct
    convolution transposed to tokens and the residual added with a rounding of its own, and bit for bit against
    convolution_ -> transposeLE_ -> add_."""
    import torch
    import juliavision_amd as jv
    x = oracle.randn_f16((N, Cin, H, W), 41)
    w = oracle.randn_f16((Cout, Cin, K, K), 42, 0, 0.05)
    b = oracle.randn_f16((Cout,), 43, 0, 0.5)
    conv = oracle.conv2d_f16(x, w, b, (s, s), (p, p), (1, 1), 1, relu)                 # (N, Cout, OH, OW)
    PQ = conv.shape[2] * conv.shape[3]
    want = np.ascontiguousarray(conv.reshape(N, Cout, PQ).transpose(0, 2, 1))
    r = None
    if res is not None:
        r = oracle.randn_f16((N if res == "each" else 1, PQ, Cout), 44)
        want = (want.astype(np.float32) + r.astype(np.float32)).astype(np.float16)
    dx, dw, db = to_dev(x), to_dev(w), to_dev(b)
    dr = None if r is None else (to_dev(r) if res == "each" else to_dev(r[0]))
    tok = poison(torch.empty((N, 1 + PQ, Cout), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.convolution_tokens_(ctx, tok[:, 1:], dx, dw, db, (s, s), (p, p), (1, 1), residual=dr, act="relu" if relu else "none")
    # the three separate ops
    chan = poison(torch.empty((N, Cout, conv.shape[2], conv.shape[3]), dtype=torch.float16, device="cuda"))
    tok2 = poison(torch.empty((N, PQ, Cout), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.convolution_(ctx, chan, dx, dw, db, (s, s), (p, p), (1, 1), 1, act="relu" if relu else "none")
    jv.transposeLE_(ctx, tok2.unsqueeze(1), chan.view(N, 1, Cout, PQ))
    if dr is not None:
        for n in range(N):
            jv.add_(ctx, tok2[n], tok2[n], dr[n] if res == "each" else dr)
    torch.cuda.synchronize()
    got = to_host(tok[:, 1:])
    assert_parity(got, want, what=f"conv -> tokens {N},{Cin},{H},{W}->{Cout} k{K} s{s} p{p} res={res}")
    if PQ > 8:            # four tokens run the decode-sized kernel, whose dot products sum in another order than the MFMA tiles
        assert np.array_equal(got, to_host(tok2))
    assert bool(torch.isnan(tok[:, 0]).all())                                         # row 0 of each image untouched


def test_conv_tokens_declines_misaligned_rows(ctx):
    import torch
    import juliavision_amd as jv
    from juliavision_amd import _lib as L
    z = lambda *sh: torch.zeros(sh, dtype=torch.float16, device="cuda")
    with pytest.raises(jv.DeclineError) as e:                                         # a row pitch of 36 halves
        jv.convolution_tokens_(ctx, z(1, 16, 36)[:, :, :32], z(1, 3, 16, 16), z(32, 3, 4, 4), None, (4, 4), (0, 0), (1, 1))
    assert e.value.status == L.DECLINE_OPERANDS


def test_conv_grouped_direct(ctx):
    _conv(ctx, 1, 8, 10, 10, 16, 3, 3, 1, 1, groups=4, expect="direct", relu=True)


def test_conv_config3_patch_embed_full(ctx):
    _conv(ctx, 1, 3, 518, 518, 384, 14, 14, 14, 0, expect="im2col_gemm", seed=5)


def test_conv_config4_full(ctx):
    """3x3 256->256 on 64x64 (M=4096, K=2304, N=256) at full size against the oracle's direct convolution on all 256
    output channels."""
    import torch
    import juliavision_amd as jv
    x = oracle.randn_f16((1, 256, 64, 64), 7)
    w = oracle.randn_f16((256, 256, 3, 3), 8, 0, 0.02)
    b = oracle.randn_f16((256,), 9, 0, 0.02)
    out = poison(torch.empty((1, 256, 64, 64), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.convolution_(ctx, out, to_dev(x), to_dev(w), to_dev(b), (1, 1), (1, 1), (1, 1), 1)
    torch.cuda.synchronize()
    got = to_host(out)
    assert np.all(np.isfinite(got))
    want = oracle.conv2d_f16(x, w, b, (1, 1), (1, 1))
    assert_parity(got, want, what="config4 conv, all channels")
    for ch in (np.r_[0:8], np.r_[248:256]):
        assert_parity(got[:, ch], want[:, ch], what=f"config4 conv channels {ch[0]}..{ch[-1]}")


def _conv_nhwc(ctx, N, Cin, H, W, Cout, KH, KW, s, p, d=1, bias=True, relu=False, seed=1):
    """The channels-last entry point against the oracle's direct convolution over the same data re-laid to
    (N,C,H,W): the layouts differ, the sums do not."""
    import torch
    import juliavision_amd as jv
    pair = lambda v: v if isinstance(v, tuple) else (v, v)
    s, p, d = pair(s), pair(p), pair(d)
    x = oracle.randn_f16((N, Cin, H, W), seed)
    w = oracle.randn_f16((Cout, Cin, KH, KW), seed + 1, 0, 0.05)
    b = oracle.randn_f16((Cout,), seed + 2, 0, 0.5) if bias else None
    want = oracle.conv2d_f16(x, w, b, s[::-1], p[::-1], d[::-1], 1, relu)
    xl, wl = np.ascontiguousarray(x.transpose(0, 2, 3, 1)), np.ascontiguousarray(w.transpose(0, 2, 3, 1))
    out = poison(torch.empty((want.shape[0], want.shape[2], want.shape[3], want.shape[1]), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.convolution_nhwc_(ctx, out, to_dev(xl), to_dev(wl), None if b is None else to_dev(b), s, p, d, act="relu" if relu else "none")
    torch.cuda.synchronize()
    assert_parity(to_host(out).transpose(0, 3, 1, 2), want, what=f"conv nhwc {N},{H},{W},{Cin}->{Cout} k{KH}x{KW} s{s} p{p} d{d}")


@pytest.mark.parametrize("N,Cin,H,W,Cout,KH,KW,s,p,d,kw", [
    (1, 256, 16, 16, 256, 3, 3, 1, 1, 1, {}),                      # config 4's 3x3 256->256 on a small map
    (2, 64, 24, 24, 104, 3, 3, 1, 1, 1, {"relu": True}),           # two images: output rows cross the image boundary inside a tile
    (1, 64, 40, 40, 64, 7, 7, 1, 3, 1, {"bias": False}),           # 49 taps, three pixels of padding on every side
    (1, 128, 20, 24, 96, 5, 5, 1, (4, 2), (2, 1), {}),             # dilation 2 along x only, unequal padding; two 64-channel runs per tap
    (1, 64, 18, 16, 48, 3, 1, (1, 2), (0, 1), 1, {}),              # 3 rows x 1 column of taps, stride 2 along y
    (3, 64, 30, 30, 256, 5, 5, 2, 2, 1, {"relu": True}),           # stride 2 both ways, M = 675: a ragged last row tile
    (1, 128, 8, 8, 64, 1, 1, 1, 0, 1, {}),                         # 1x1: the gather degenerates to a plain row-major operand
    (1, 192, 12, 32, 32, 1, 3, 1, (1, 0), 1, {}),                  # KH = 1, KW = 3, three runs per tap
    (5, 64, 3, 3, 8, 3, 3, 1, 0, 1, {}),                           # one output pixel per image, M = 5
    (1, 512, 32, 32, 128, 3, 3, 1, 1, 1, {"relu": True}),          # K = 4608 over eight output tiles: split into fp32 planes
])
def test_conv_nhwc(ctx, N, Cin, H, W, Cout, KH, KW, s, p, d, kw):
    _conv_nhwc(ctx, N, Cin, H, W, Cout, KH, KW, s, p, d, **kw)


def test_conv_nhwc_config4_is_the_nchw_result(ctx):
    """3x3 256->256 on 64x64 at full size (M=4096, K=2304, N=256): the oracle checks 16 output channels,
    the reference-layout path checks the rest (same products, summed in a different order: fp16 rounding apart)."""
    import torch
    import juliavision_amd as jv
    x = oracle.randn_f16((1, 256, 64, 64), 7)
    w = oracle.randn_f16((256, 256, 3, 3), 8, 0, 0.02)
    b = oracle.randn_f16((256,), 9, 0, 0.02)
    dx, dw, db = to_dev(x), to_dev(w), to_dev(b)
    out = poison(torch.empty((1, 64, 64, 256), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.convolution_nhwc_(ctx, out, dx.permute(0, 2, 3, 1).contiguous(), dw.permute(0, 2, 3, 1).contiguous(), db, (1, 1), (1, 1), (1, 1))
    ref = poison(torch.empty((1, 256, 64, 64), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.convolution_(ctx, ref, dx, dw, db, (1, 1), (1, 1), (1, 1), 1)
    torch.cuda.synchronize()
    got = to_host(out).transpose(0, 3, 1, 2)
    ch = np.r_[0:8, 248:256]
    assert_parity(got[:, ch], oracle.conv2d_f16(x, w[ch], b[ch], (1, 1), (1, 1)), what="config4 nhwc conv band")
    assert_parity(got, to_host(ref), what="config4 nhwc vs nchw")


def test_conv_nhwc_declines(ctx):
    import torch
    import juliavision_amd as jv
    from juliavision_amd import _lib as L
    f = lambda *sh: torch.zeros(sh, dtype=torch.float16, device="cuda")
    with pytest.raises(jv.DeclineError) as e:      # 32 channels: not a whole 64-channel run
        jv.convolution_nhwc_(ctx, f(1, 8, 8, 64), f(1, 8, 8, 32), f(64, 3, 3, 32), None, (1, 1), (1, 1), (1, 1))
    assert e.value.status == L.DECLINE_UNSUPPORTED
    with pytest.raises(jv.DeclineError) as e:      # output of the wrong extent
        jv.convolution_nhwc_(ctx, f(1, 8, 8, 64), f(1, 8, 8, 64), f(64, 3, 3, 64), None, (2, 2), (1, 1), (1, 1))
    assert e.value.status == L.DECLINE_OPERANDS


def _convt(ctx, N, Cin, H, W, Cout, KH, KW, s, p=0, d=1, op=0, groups=1, bias=True, expect=None, seed=1):
    """``s``, ``p``, ``d``, ``op``: one number for both axes or an ``(x, y)`` pair."""
    import torch
    import juliavision_amd as jv
    pair = lambda v: v if isinstance(v, tuple) else (v, v)
    s, p, d, op = pair(s), pair(p), pair(d), pair(op)
    x = oracle.randn_f16((N, Cin, H, W), seed, 0, 0.5)
    w = oracle.randn_f16((Cin, Cout // groups, KH, KW), seed + 1, 0, 0.05)
    b = oracle.randn_f16((Cout,), seed + 2, 0, 0.5) if bias else None
    want = oracle.convtranspose2d_f16(x, w, b, s[::-1], p[::-1], d[::-1], op[::-1], groups)
    out = poison(torch.empty(want.shape, dtype=torch.float16, device="cuda"))
    dx, dw = to_dev(x), to_dev(w)
    plan = jv.convtranspose_plan(ctx.dev, out, dx, dw, s, p, d, op, groups)
    if expect:
        assert plan.path == expect, plan
    ctx.ws.reset()
    jv.convolutiontranspose_(ctx, out, dx, dw, None if b is None else to_dev(b), s, p, d, op, groups)
    torch.cuda.synchronize()
    got = to_host(out)
    assert_parity(got, want, what=f"convT {N},{Cin},{H},{W}->{Cout} k{KH}x{KW} s{s} p{p} d{d} op{op} g{groups}")
    return got, want


@pytest.mark.parametrize("N,Cin,H,W,Cout,KH,KW,kw", [
    (1, 256, 64, 64, 64, 2, 2, {}),                   # SAM 2's two upsamplers, test_convtranspose_gemm.jl:36
    (1, 64, 128, 128, 32, 2, 2, {}),
    (1, 32, 16, 16, 8, 2, 2, {}),                     # channel counts below the GEMM tile
    (2, 24, 8, 8, 12, 2, 2, {"bias": False}),
    (3, 40, 5, 7, 10, 3, 2, {}),                      # H*W = 35 and OW = 14: the unaligned GEMM and the scalar shuffle
    (1, 48, 6, 8, 16, 1, 4, {}),                      # one row of taps
    (1, 16, 12, 12, 24, 1, 1, {}),                    # 1x1 stride 1: a plain channel mix
])
def test_convtranspose_gemm_shuffle(ctx, N, Cin, H, W, Cout, KH, KW, kw):
    got, _ = _convt(ctx, N, Cin, H, W, Cout, KH, KW, (KW, KH), expect="gemm_shuffle", **kw)
    # a shuffle that drops a sub-pixel phase leaves a lattice of zeros that an averaged error would hide
    # (test_convtranspose_gemm.jl:50-58)
    for ky in range(KH):
        for kx in range(KW):
            assert np.any(got[:, :, ky::KH, kx::KW] != 0)


@pytest.mark.parametrize("N,Cin,H,W,Cout,KH,KW,s,p,d,op,g", [
    (1, 16, 8, 8, 8, 3, 3, 2, 0, 1, 0, 1),                         # test_convtranspose_gemm.jl:78-95: overlapping fields
    (2, 6, 5, 7, 4, 2, 3, (3, 2), (0, 1), (2, 1), (2, 1), 2),      # everything unequal, two groups
    (1, 8, 6, 6, 8, 4, 4, 2, 1, 1, 0, 8),                          # depthwise 4/2/1 upsampler
    (1, 3, 1, 9, 5, 1, 5, (3, 1), (2, 0), 1, (2, 0), 1),           # a lifted 1-D layer
    (1, 16, 8, 8, 8, 2, 2, 2, 0, 1, 1, 1),                         # kernel == stride but with output padding
])
def test_convtranspose_gather(ctx, N, Cin, H, W, Cout, KH, KW, s, p, d, op, g):
    _convt(ctx, N, Cin, H, W, Cout, KH, KW, s, p, d, op, g, expect="gather")


def test_convtranspose_routes_agree_bitwise_on_exact_data(ctx):
    """Small integers make every product and sum exact in fp16/fp32, so the GEMM + shuffle route, the gather
    kernel and the oracle must agree bit for bit whatever their summation order."""
    import torch
    import juliavision_amd as jv
    rng = np.random.default_rng(3)
    x = rng.integers(-3, 4, (2, 32, 8, 16)).astype(np.float16)
    w = rng.integers(-2, 3, (32, 12, 2, 2)).astype(np.float16)
    b = rng.integers(-4, 5, (12,)).astype(np.float16)
    want = oracle.convtranspose2d_f16(x, w, b, (2, 2))
    out = poison(torch.empty(want.shape, dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.convolutiontranspose_(ctx, out, to_dev(x), to_dev(w), to_dev(b), (2, 2), (0, 0), (1, 1), (0, 0), 1)
    assert np.array_equal(to_host(out), want)
    # the same numbers through the gather: two groups of half the channels, summed by hand, is not the same op,
    # so reach the gather with an output padding instead and compare the part both produce
    want_op = oracle.convtranspose2d_f16(x, w, b, (2, 2), output_padding=(1, 1))
    out_op = poison(torch.empty(want_op.shape, dtype=torch.float16, device="cuda"))
    jv.convolutiontranspose_(ctx, out_op, to_dev(x), to_dev(w), to_dev(b), (2, 2), (0, 0), (1, 1), (1, 1), 1)
    got_op = to_host(out_op)
    assert np.array_equal(got_op, want_op)
    assert np.array_equal(got_op[:, :, :-1, :-1], want)
    assert np.array_equal(got_op[:, :, -1, :], np.broadcast_to(b[None, :, None], (2, 12, 33)))   # the padded edge is the bias


@pytest.mark.parametrize("groups,C", [(1500, 1280), (1370, 384), (7, 144), (5, 37), (3, 4096), (2, 5000)])
@pytest.mark.parametrize("affine", [True, False])
def test_layernorm(ctx, groups, C, affine):
    import torch
    import juliavision_amd as jv
    a = oracle.randn_f16((groups, C), 3, 0.3, 2.0)
    g = oracle.randn_f16((C,), 4, 1.0, 0.1) if affine else None
    b = oracle.randn_f16((C,), 5, 0.0, 0.1) if affine else None
    want, mu, rs = oracle.layernorm_f16(a, g, b, 1e-5)
    out = poison(torch.empty((groups, C), dtype=torch.float16, device="cuda"))
    mean = torch.empty(groups, dtype=torch.float32, device="cuda")
    rstd = torch.empty(groups, dtype=torch.float32, device="cuda")
    jv.layernorm_(ctx, out, mean, rstd, to_dev(a), None if g is None else to_dev(g), None if b is None else to_dev(b), C, 1e-5)
    torch.cuda.synchronize()
    assert_parity(to_host(out), want, what=f"layernorm {groups}x{C}")
    np.testing.assert_allclose(to_host(mean), mu, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(to_host(rstd), rs, rtol=1e-4, atol=1e-6)


def test_add_bit_exact(ctx):
    import torch
    import juliavision_amd as jv
    for n in (1500 * 1280, 1001):
        a = oracle.randn_f16((n,), 1)
        b = oracle.randn_f16((n,), 2)
        out = torch.empty(n, dtype=torch.float16, device="cuda")
        jv.add_(ctx, out, to_dev(a), to_dev(b))
        torch.cuda.synchronize()
        assert np.array_equal(to_host(out).view(np.uint16), oracle.add_f16(a, b).view(np.uint16))


@pytest.mark.parametrize("B,H,Ln,E", [(1, 1, 384, 1369), (2, 3, 70, 64), (1, 20, 33, 65), (1, 2, 1, 40), (3, 1, 50, 1)])
@pytest.mark.parametrize("source", ["dense", "token_major", "already_l_fastest"])
def test_transpose_le_moves_bits(ctx, B, H, Ln, E, source):
    """(E,L,H,B) strided -> dense (L,E,H,B), the contract of transposeLE (attention.jl:374-396); exact."""
    import torch
    import juliavision_amd as jv
    vals = oracle.randn_f16((B, H, Ln, E), 17)
    if source == "dense":
        a = to_dev(vals)
    elif source == "token_major":                     # a (B,L,H,E) buffer seen as (B,H,L,E): heads are column bands of token rows
        a = to_dev(np.ascontiguousarray(vals.transpose(0, 2, 1, 3))).permute(0, 2, 1, 3)
    else:                                             # memory already runs along l: the strided-copy kernel
        a = to_dev(np.ascontiguousarray(vals.transpose(0, 1, 3, 2))).permute(0, 1, 3, 2)
    assert np.array_equal(to_host(a), vals)
    out = poison(torch.empty((B, H, E, Ln), dtype=torch.float16, device="cuda"))
    jv.transposeLE_(ctx, out, a)
    assert np.array_equal(to_host(out), vals.transpose(0, 1, 3, 2))
    # into a wider destination: rows of a larger matrix, the columns beside them untouched
    wide = poison(torch.empty((B, H, E, Ln + 5), dtype=torch.float16, device="cuda"))
    jv.transposeLE_(ctx, wide[..., 2:2 + Ln], a)
    got = to_host(wide)
    assert np.array_equal(got[..., 2:2 + Ln], vals.transpose(0, 1, 3, 2)) and np.all(np.isnan(got[..., :2])) and np.all(np.isnan(got[..., 2 + Ln:]))


def test_transpose_le_2d_is_the_matrix_transpose(ctx):
    import torch
    import juliavision_amd as jv
    w = oracle.randn_f16((100, 37), 3)
    out = poison(torch.empty((37, 100), dtype=torch.float16, device="cuda"))
    jv.transposeLE_(ctx, out, to_dev(w))
    assert np.array_equal(to_host(out), w.T)


@pytest.mark.parametrize("rows,n,scale", [(7, 64, 1.0), (5, 37, 1.0), (9, 1370, 0.125), (6, 1376, 0.125), (3, 4096, 1.0), (2, 5000, 0.5)])
def test_softmax_rows(ctx, rows, n, scale):
    """softmax_kernel! (ops.jl:474-573) / attn_softmax_rows! (attention.jl:528-615): register-resident rows up to 4096,
    the three-pass form beyond and for rows that are not 16-byte addressable."""
    import torch
    import juliavision_amd as jv
    a = oracle.randn_f16((rows, n), 21, std=3.0)
    a[rows // 2, : n // 3] = -np.inf                      # masked keys: weight exactly 0
    out = poison(torch.empty((rows, n), dtype=torch.float16, device="cuda"))
    jv.softmax_(ctx, out, to_dev(a), scale)
    torch.cuda.synchronize()
    got = to_host(out)
    assert np.all(got[rows // 2, : n // 3] == 0)
    assert_parity(got, oracle.softmax_f16(a, scale), what=f"softmax {rows}x{n}")
    assert np.allclose(got.astype(np.float64).sum(-1), 1.0, atol=4e-3)


def test_softmax_fp32_rows_and_a_fully_masked_row(ctx):
    import torch
    import juliavision_amd as jv
    a = oracle.randn_f32((4, 300), 22, std=4.0)
    a[1] = -np.inf
    out = poison(torch.empty((4, 300), dtype=torch.float32, device="cuda"))
    jv.softmax_(ctx, out, to_dev(a))
    torch.cuda.synchronize()
    got = to_host(out)
    x = a.astype(np.float64)[[0, 2, 3]]
    e = np.exp(x - x.max(-1, keepdims=True))
    assert np.all(got[1] == 0) and np.max(np.abs(got[[0, 2, 3]] - e / e.sum(-1, keepdims=True))) < 1e-6


def test_scale_bit_exact(ctx):
    import torch
    import juliavision_amd as jv
    a = oracle.randn_f16((3, 1001), 23, std=5.0)
    out = poison(torch.empty((3, 1001), dtype=torch.float16, device="cuda"))
    jv.scale_(ctx, out, to_dev(a), 0.125)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(out).view(np.uint16), oracle.scale_f16(a, 0.125).view(np.uint16))
    jv.scale_(ctx, out, to_dev(a), 1.0 / 3.0)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(out).view(np.uint16), oracle.scale_f16(a, 1.0 / 3.0).view(np.uint16))


@pytest.mark.parametrize("kind", ["gelu", "gelu_tanh", "relu"])
def test_standalone_activation_is_the_epilogue_function(ctx, kind):
    """The activation on its own gives what the GEMM epilogue gives: the oracle's erf / tanh / relu forms
    (ops.jl:161-169, 1665-1685) on fp16 values, one rounding."""
    import torch
    import juliavision_amd as jv
    a = np.concatenate([oracle.randn_f16((2000,), 31, std=2.5), np.arange(-8, 8, 0.01).astype(np.float16)])
    out = poison(torch.empty(a.shape, dtype=torch.float16, device="cuda"))
    jv.act_(ctx, out, to_dev(a), kind)
    torch.cuda.synchronize()
    got, want = to_host(out).astype(np.float64), oracle.act_f16(a, kind).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2e-3 * max(1.0, np.max(np.abs(want)))        # device exp / rcp against libm: an ulp of fp16
    assert_parity(got, want, what=kind)
    # the ends of the fp16 range: a linear whose sum overflowed hands the activation +-65504 or +inf, and the
    # reference's expression returns them unchanged on the positive side and (signed) zero on the negative
    edge = np.array([6.0, 14.0, 100.0, 1000.0, 65504.0, np.inf, -6.0, -14.0, -100.0, -1000.0, -65504.0], dtype=np.float16)
    out = poison(torch.empty(edge.shape, dtype=torch.float16, device="cuda"))
    jv.act_(ctx, out, to_dev(edge), kind)
    torch.cuda.synchronize()
    got, want = to_host(out), oracle.act_f16(edge, kind)
    assert not np.isnan(got).any(), got
    assert np.array_equal(got[3:6], want[3:6]) and np.array_equal(np.abs(got[7:]), np.abs(want[7:])), (got, want)
    assert np.allclose(got.astype(np.float64)[:3], want.astype(np.float64)[:3], rtol=2e-3)


def test_clamp_bit_exact(ctx):
    import torch
    import juliavision_amd as jv
    a = oracle.randn_f16((4099,), 32, std=3e4)            # many values beyond the guard
    a[:3] = [np.inf, -np.inf, 65504.0]
    out = poison(torch.empty(a.shape, dtype=torch.float16, device="cuda"))
    jv.clamp_(ctx, out, to_dev(a), -64504.0, 64504.0)
    torch.cuda.synchronize()
    want = np.clip(a.astype(np.float32), -64504.0, 64504.0).astype(np.float16)
    assert np.array_equal(to_host(out).view(np.uint16), want.view(np.uint16))


def test_rowwise_entry_points_decline_bad_arguments(ctx):
    """Status codes of the row-wise glue: nothing is launched for a null operand, an empty or negative extent, an
    unknown activation or an inverted clamp interval."""
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    a = torch.zeros(64, dtype=torch.float16, device="cuda")
    p, st = a.data_ptr(), ctx.stream
    assert lib.mi_softmax_f16(None, p, L.F16, 8, 8, 1.0, st) == L.DECLINE_OPERANDS
    assert lib.mi_softmax_f16(p, p, 7, 8, 8, 1.0, st) == L.DECLINE_OPERANDS          # neither fp16 nor fp32
    assert lib.mi_softmax_f16(p, p, L.F16, 0, 8, 1.0, st) == L.DECLINE_EXTENT
    assert lib.mi_softmax_f16(p, p, L.F16, 8, 0, 1.0, st) == L.OK                     # no rows: nothing to do
    assert lib.mi_scale_f16(p, None, 2.0, 64, st) == L.DECLINE_OPERANDS
    assert lib.mi_scale_f16(p, p, 2.0, -1, st) == L.DECLINE_EXTENT
    assert lib.mi_act_f16(p, p, 9, 64, st) == L.DECLINE_UNSUPPORTED
    assert lib.mi_clamp_f16(p, p, 1.0, -1.0, 64, st) == L.DECLINE_EXTENT
    assert lib.mi_clamp_f16(p, p, float("nan"), 1.0, 64, st) == L.DECLINE_EXTENT
    torch.cuda.synchronize()
    assert bool((a == 0).all())
