"""Decode-step plumbing on the GPU: the in-place KV-cache write, a decoder-layer step against a
CPU composition of the oracle's kernels, and graph replay against the eager step."""
import numpy as np
import pytest

import oracle
from util import assert_parity, poison, to_dev, to_host

pytestmark = pytest.mark.gpu


def _weights(d, ffn, seed, layout):
    """Random decoder-layer weights: numpy [K][F] masters plus device tensors in the asked layout."""
    import torch
    from juliavision_amd.decode import DecoderLayerWeights
    host, dev = {}, {}
    shapes = {"wqkv": (d, 3 * d), "wo": (d, d), "wq_c": (d, d), "wo_c": (d, d), "w1": (d, ffn), "w2": (ffn, d)}
    for i, (name, (k, f)) in enumerate(shapes.items()):
        w = oracle.randn_f16((k, f), seed + i, std=0.05)
        host[name] = w
        dev[name] = to_dev(w) if layout == "kf" else to_dev(np.ascontiguousarray(w.T)).t()
    for i, (name, n) in enumerate({"bqkv": 3 * d, "bo": d, "bq_c": d, "bo_c": d, "b1": ffn, "b2": d}.items()):
        host[name] = oracle.randn_f16((n,), seed + 20 + i, std=0.02)
        dev[name] = to_dev(host[name])
    for i, name in enumerate(["ln1", "ln2", "ln3"]):
        host[name + "_g"] = oracle.randn_f16((d,), seed + 40 + i, mean=1.0, std=0.1)
        host[name + "_b"] = oracle.randn_f16((d,), seed + 50 + i, std=0.1)
        dev[name + "_g"], dev[name + "_b"] = to_dev(host[name + "_g"]), to_dev(host[name + "_b"])
    return host, DecoderLayerWeights(**dev)


def _oracle_layer_step(Wh, x, self_k, self_v, cross_k, cross_v, length, H, E):
    """The same layer step from the oracle's CPU kernels; self_k/self_v (B,H,Lmax,E) are updated in place,
    ``length`` (B,) counts the live slots including the new one; Lmax + 1 marks a row stepped while full, whose
    new K/V is not stored and which attends over the Lmax stored keys."""
    B, d = x.shape
    h, _, _ = oracle.layernorm_f16(x, Wh["ln1_g"], Wh["ln1_b"])
    qkv = oracle.gemm_f16(h, Wh["wqkv"], Wh["bqkv"])
    q, k, v = (qkv[:, i * d:(i + 1) * d].reshape(B, H, 1, E) for i in range(3))
    for b in range(B):
        if 1 <= length[b] <= self_k.shape[2]:
            self_k[b, :, length[b] - 1, :] = k[b, :, 0, :]
            self_v[b, :, length[b] - 1, :] = v[b, :, 0, :]
    att = oracle.sdpa_threepass_f16(np.ascontiguousarray(q), self_k, self_v, kv_len=np.minimum(length, self_k.shape[2]).astype(np.int32))
    x1 = oracle.gemm_f16(att.reshape(B, d), Wh["wo"], Wh["bo"], residual=x)
    h, _, _ = oracle.layernorm_f16(x1, Wh["ln2_g"], Wh["ln2_b"])
    qc = oracle.gemm_f16(h, Wh["wq_c"], Wh["bq_c"]).reshape(B, H, 1, E)
    catt = oracle.sdpa_threepass_f16(qc, cross_k, cross_v)
    x2 = oracle.gemm_f16(catt.reshape(B, d), Wh["wo_c"], Wh["bo_c"], residual=x1)
    h, _, _ = oracle.layernorm_f16(x2, Wh["ln3_g"], Wh["ln3_b"])
    f = oracle.gemm_f16(h, Wh["w1"], Wh["b1"], epi="gelu")
    return oracle.gemm_f16(f, Wh["w2"], Wh["b2"], residual=x2)


@pytest.mark.parametrize("E", [64, 12])
def test_kv_append_writes_one_slot_per_row(ctx, E):
    import torch
    from juliavision_amd.decode import KVCache
    B, H, Lmax = 4, 3, 16
    cache = KVCache(2, B, H, E, max_target=Lmax, src_len=8)
    before_k = oracle.randn_f16((2, B, H, Lmax, E), 7)
    before_v = oracle.randn_f16((2, B, H, Lmax, E), 8)
    cache.self_k.copy_(to_dev(before_k))
    cache.self_v.copy_(to_dev(before_v))
    cache.length.copy_(torch.tensor([1, 5, 16, 0], dtype=torch.int32))
    # the new rows sit inside a wider buffer, as the q/k/v thirds of a projection do
    wide_k = to_dev(oracle.randn_f16((B, 3 * H * E), 9))
    k_new = wide_k[:, H * E:2 * H * E].unflatten(1, (H, 1, E))
    v_new = to_dev(oracle.randn_f16((B, 3 * H * E), 10))[:, 2 * H * E:].unflatten(1, (H, 1, E))
    cache.append(ctx, 1, k_new, v_new)
    torch.cuda.synchronize()
    want_k, want_v = before_k.copy(), before_v.copy()
    kn, vn = to_host(k_new), to_host(v_new)
    for b, n in enumerate([1, 5, 16, 0]):
        if n >= 1:
            want_k[1, b, :, n - 1, :] = kn[b, :, 0, :]
            want_v[1, b, :, n - 1, :] = vn[b, :, 0, :]
    assert np.array_equal(to_host(cache.self_k), want_k)      # bit-exact, and nothing else touched
    assert np.array_equal(to_host(cache.self_v), want_v)


def test_kv_advance_clamps(ctx):
    import torch
    from juliavision_amd.decode import KVCache
    cache = KVCache(1, 5, 1, 8, max_target=4, src_len=1)
    cache.length.copy_(torch.tensor([0, 1, 3, 4, 2], dtype=torch.int32))
    cache.advance(ctx)
    assert to_host(cache.length).tolist() == [1, 2, 4, 5, 3]      # capacity + 1: "this row was stepped while full"
    assert cache.overflowed()
    cache.advance(ctx)
    assert to_host(cache.length).tolist() == [2, 3, 5, 5, 4]      # and there it stops
    cache.advance(ctx, -4)
    assert to_host(cache.length).tolist() == [0, 0, 1, 1, 0]
    assert not cache.overflowed()


@pytest.mark.parametrize("layout", ["kf", "fk"])
@pytest.mark.parametrize("B", [1, 4])
def test_decoder_layer_steps_match_oracle(ctx, B, layout):
    import torch
    from juliavision_amd.decode import DecodeBuffers, KVCache, decoder_layer_step
    d, H, E, ffn, Lmax, Ls = 256, 4, 64, 512, 12, 70
    Wh, Wd = _weights(d, ffn, 100, layout)
    cache = KVCache(1, B, H, E, max_target=Lmax, src_len=Ls)
    ck = oracle.randn_f16((1, B, H, Ls, E), 31)
    cv = oracle.randn_f16((1, B, H, Ls, E), 32)
    cache.cross_k.copy_(to_dev(ck))
    cache.cross_v.copy_(to_dev(cv))
    start = np.array([0, 3, 7, 11][:B], dtype=np.int32)          # ragged histories, one row about to fill up
    hk = np.zeros((B, H, Lmax, E), dtype=np.float16)
    hv = np.zeros((B, H, Lmax, E), dtype=np.float16)
    for b in range(B):
        hk[b, :, :start[b]] = oracle.randn_f16((H, start[b], E), 40 + b)
        hv[b, :, :start[b]] = oracle.randn_f16((H, start[b], E), 50 + b)
    cache.self_k[0].copy_(to_dev(hk))
    cache.self_v[0].copy_(to_dev(hv))
    cache.length.copy_(to_dev(start))
    buf = DecodeBuffers(B, d, ffn)
    out = torch.empty((B, d), dtype=torch.float16, device="cuda")
    length = start.copy()
    for step in range(3):
        x = oracle.randn_f16((B, d), 60 + step)
        cache.advance(ctx)
        out.fill_(float("nan"))
        decoder_layer_step(ctx, Wd, cache, 0, to_dev(x), out, buf)
        length = np.minimum(length + 1, Lmax + 1)
        want = _oracle_layer_step(Wh, x, hk, hv, ck[0], cv[0], length, H, E)
        assert_parity(to_host(out), want, what=f"decoder layer B{B} {layout} step {step}")
        assert to_host(cache.length).tolist() == length.tolist()
        # the cache rows written on the device are the oracle's rows (fp16 outputs of the same GEMV, within rounding)
        assert_parity(to_host(cache.self_k[0]), hk, what=f"self_k after step {step}")


def test_weights_relaid_at_load_run_the_one_launch_linears(ctx):
    """DecoderLayerWeights.k_contiguous: [K][F] weights re-laid once to [F][K] hold the same values, and a layer step
    over them gives the bits of a step over weights that were [F][K] from the start."""
    import torch
    from juliavision_amd.decode import DecodeBuffers, KVCache, decoder_layer_step
    B, d, H, E, ffn = 2, 256, 4, 64, 512
    _, Wkf = _weights(d, ffn, 100, "kf")
    _, Wfk = _weights(d, ffn, 100, "fk")
    Wre = Wkf.k_contiguous(ctx)
    torch.cuda.synchronize()
    for name in Wkf.LINEARS:
        a, b = getattr(Wre, name), getattr(Wkf, name)
        assert a.stride(0) == 1 and a.shape == b.shape and bool((a == b).all()), name
        assert getattr(Wfk.k_contiguous(ctx), name) is getattr(Wfk, name)          # nothing to do: kept
    outs = []
    for W in (Wre, Wfk):
        cache = KVCache(1, B, H, E, max_target=16, src_len=40)
        cache.cross_k.copy_(to_dev(oracle.randn_f16((1, B, H, 40, E), 31)))
        cache.cross_v.copy_(to_dev(oracle.randn_f16((1, B, H, 40, E), 32)))
        buf, out = DecodeBuffers(B, d, ffn), poison(torch.empty((B, d), dtype=torch.float16, device="cuda"))
        cache.advance(ctx)
        decoder_layer_step(ctx, W, cache, 0, to_dev(oracle.randn_f16((B, d), 60)), out, buf)
        torch.cuda.synchronize()
        outs.append(to_host(out))
    assert np.isfinite(outs[0]).all() and np.array_equal(outs[0], outs[1])


def test_step_graph_replays_match_eager(ctx):
    """One captured step (advance + two layers) replayed over advancing positions, with eager work and
    synchronisation between replays; every replay equals an eager twin bit for bit."""
    import torch
    from juliavision_amd import kernels as K
    from juliavision_amd.decode import DecodeBuffers, KVCache, StepGraph, decoder_layer_step
    B, d, H, E, ffn, Lmax, Ls, NL = 2, 256, 4, 64, 512, 16, 40, 2
    layers = [_weights(d, ffn, 200 + 100 * i, "kf")[1] for i in range(NL)]

    def make_state():
        cache = KVCache(NL, B, H, E, max_target=Lmax, src_len=Ls)
        cache.cross_k.copy_(to_dev(oracle.randn_f16((NL, B, H, Ls, E), 71)))
        cache.cross_v.copy_(to_dev(oracle.randn_f16((NL, B, H, Ls, E), 72)))
        return cache, DecodeBuffers(B, d, ffn), torch.zeros((B, d), dtype=torch.float16, device="cuda"), \
            [torch.empty((B, d), dtype=torch.float16, device="cuda") for _ in range(NL)]

    def step(cache, buf, x, outs):
        cache.advance(ctx)
        src = x
        for i in range(NL):
            decoder_layer_step(ctx, layers[i], cache, i, src, outs[i], buf)
            src = outs[i]

    cg, bg, xg, og = make_state()
    ce, be, xe, oe = make_state()
    graph = StepGraph(lambda: step(cg, bg, xg, og), restore=lambda: (cg.reset(), cg.self_k.zero_(), cg.self_v.zero_()))
    side_a = to_dev(oracle.randn_f16((64, 64), 5))
    side_y = torch.empty((64, 64), dtype=torch.float16, device="cuda")
    for t in range(5):
        x = to_dev(oracle.randn_f16((B, d), 300 + t))
        xg.copy_(x)
        xe.copy_(x)
        graph.replay()
        step(ce, be, xe, oe)
        K.matmul_(ctx, side_y, side_a, side_a)          # the program's own eager work between replays
        torch.cuda.synchronize()
        assert np.array_equal(to_host(og[-1]), to_host(oe[-1])), f"replay {t} differs from the eager step"
        assert np.array_equal(to_host(cg.self_k), to_host(ce.self_k))
        assert to_host(cg.length).tolist() == [t + 1] * B


@pytest.mark.parametrize("E,Lmax", [(64, 448), (32, 70), (64, 16), (64, 1500), (48, 2049), (64, 8000)])
def test_fused_append_and_attend_equals_the_two_calls(ctx, E, Lmax):
    """mi_sdpa_append_f16 against mi_kv_append_f16 followed by mi_sdpa_f16 on a twin cache: the same cache bits, the
    same output bits (both attend with the one-launch kernel, its key range cut over the same number of workgroups),
    and the oracle's attention over the updated cache."""
    import torch
    import juliavision_amd as jv
    B, H = 4, 3
    lens = [1, 5, Lmax, 0]
    hk, hv = oracle.randn_f16((B, H, Lmax, E), 11), oracle.randn_f16((B, H, Lmax, E), 12)
    wide = to_dev(oracle.randn_f16((B, 3 * H * E), 13))                 # q, k, v as column bands of one projection
    q, k_new, v_new = (wide[:, i * H * E:(i + 1) * H * E].unflatten(1, (H, 1, E)) for i in range(3))
    length = torch.tensor(lens, dtype=torch.int32, device="cuda")
    ck1, cv1, ck2, cv2 = to_dev(hk), to_dev(hv), to_dev(hk), to_dev(hv)
    out1 = torch.full((B, H, 1, E), float("nan"), dtype=torch.float16, device="cuda")
    out2 = out1.clone()
    jv.sdpa_append(ctx, q, ck1, cv1, k_new, v_new, length, out=out1)
    strides = lambda t: jv.kernels._strides_elbh(t)
    rc = jv._lib.init().mi_kv_append_f16(ck2.data_ptr(), cv2.data_ptr(), strides(ck2), Lmax, k_new.data_ptr(), v_new.data_ptr(),
                                         strides(k_new), length.data_ptr(), E, H, B, ctx.stream)
    assert rc == 0
    ctx.ws.reset()
    jv.sdpa(ctx, q, ck2, cv2, out=out2, kv_len=length)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(ck1), to_host(ck2)) and np.array_equal(to_host(cv1), to_host(cv2))
    assert np.array_equal(to_host(out1), to_host(out2))
    assert np.all(to_host(out1)[3] == 0)                               # no live key: zeros, and nothing appended
    assert np.array_equal(to_host(ck1)[3], hk[3])
    want = oracle.sdpa_threepass_f16(to_host(q), to_host(ck1), to_host(cv1), kv_len=np.array(lens, dtype=np.int32))
    assert_parity(to_host(out1), want, what=f"fused append + attention E{E} Lmax{Lmax}")


def test_fused_append_declines_what_the_one_launch_kernel_does_not_cover(ctx):
    import torch
    import juliavision_amd as jv
    from juliavision_amd import _lib as L
    B, H, E, Lmax = 1, 2, 128, 64                                       # head dim over 64
    z = lambda *s: torch.zeros(s, dtype=torch.float16, device="cuda")
    with pytest.raises(jv.DeclineError) as e:
        jv.sdpa_append(ctx, z(B, H, 1, E), z(B, H, Lmax, E), z(B, H, Lmax, E), z(B, H, 1, E), z(B, H, 1, E),
                       torch.ones((B,), dtype=torch.int32, device="cuda"), out=z(B, H, 1, E))
    assert e.value.status == L.DECLINE_UNSUPPORTED


@pytest.mark.parametrize("layout", ["kf", "fk"])
@pytest.mark.parametrize("B,S,H,E", [(1, 200, 4, 64), (2, 77, 3, 32)])
def test_fill_cross_writes_the_projections_head_major(ctx, B, S, H, E, layout):
    """fillcross! (decode.jl:173-177): cross K/V of a layer = the encoder output through k_proj (no bias in Whisper) and
    v_proj, laid out (B,H,S,E).  Checked against the oracle's GEMM re-laid on the host; the other layer stays untouched."""
    import torch
    from juliavision_amd.decode import KVCache
    d = H * E
    enc = oracle.randn_f16((B, S, d), 3)
    wk, wv = oracle.randn_f16((d, d), 4, std=0.05), oracle.randn_f16((d, d), 5, std=0.05)
    bv = oracle.randn_f16((d,), 6, std=0.1)
    dev_w = lambda w: to_dev(w) if layout == "kf" else to_dev(np.ascontiguousarray(w.T)).t()
    cache = KVCache(2, B, H, E, max_target=8, src_len=S)
    cache.cross_k.fill_(7.0)
    cache.cross_v.fill_(7.0)
    cache.fill_cross(ctx, 1, to_dev(enc), dev_w(wk), None, dev_w(wv), to_dev(bv))
    torch.cuda.synchronize()
    for store, w, bias in ((cache.cross_k, wk, None), (cache.cross_v, wv, bv)):
        got = to_host(store)
        assert np.all(got[0] == np.float16(7.0))
        for b in range(B):
            want = oracle.gemm_f16(enc[b], w, bias).reshape(S, H, E).transpose(1, 0, 2)
            assert_parity(got[1, b], want, what=f"fill_cross batch {b}")
