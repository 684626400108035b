"""The five benchmark configurations as whole compositions at their real sizes, through the host
mirror and the C ABI, against the same compositions of the oracle's CPU kernels: the encoder block
(1500 x 1280, 20 x 64 heads, FFN 5120), the ViT-S/14 encoder at 518 x 518 (patch embedding as
convolution-as-GEMM, 1370 tokens, 12 layers), and the decoder layer step at batch 1/4/8 over a
448-slot cache and 1500 encoder states.  The single linear and the 4096-token attention + 3x3
convolution have their full-size tests beside the kernels they exercise."""
import numpy as np
import pytest

import oracle
from util import assert_parity, poison, to_dev, to_host

pytestmark = pytest.mark.gpu


def _layer(d, ffn, seed, wstd=0.02):
    """Random pre-LN block weights: numpy [K][F] masters and the device dataclass."""
    from juliavision_amd.encoder import EncoderLayerWeights
    h = {}
    for i, (n, shape) in enumerate({"wqkv": (d, 3 * d), "wo": (d, d), "w1": (d, ffn), "w2": (ffn, d)}.items()):
        h[n] = oracle.randn_f16(shape, seed + i, 0, wstd)
    for i, (n, m) in enumerate({"bqkv": 3 * d, "bo": d, "b1": ffn, "b2": d}.items()):
        h[n] = oracle.randn_f16((m,), seed + 10 + i, 0, 0.02)
    for i, n in enumerate(("ln1", "ln2")):
        h[n + "_g"] = oracle.randn_f16((d,), seed + 20 + i, 1.0, 0.02)
        h[n + "_b"] = oracle.randn_f16((d,), seed + 30 + i, 0.0, 0.02)
    return h, EncoderLayerWeights(**{k: to_dev(v) for k, v in h.items()})


def _oracle_layer(h, x, heads, eps):
    T, d = x.shape
    E = d // heads
    n1, _, _ = oracle.layernorm_f16(x, h["ln1_g"], h["ln1_b"], eps)
    qkv = oracle.gemm_f16(n1, h["wqkv"], h["bqkv"])
    q, k, v = (np.ascontiguousarray(qkv[:, i * d:(i + 1) * d].reshape(T, heads, E).transpose(1, 0, 2))[None] for i in range(3))
    att = oracle.sdpa_threepass_f16(q, k, v)[0].transpose(1, 0, 2).reshape(T, d)
    x1 = oracle.gemm_f16(np.ascontiguousarray(att), h["wo"], h["bo"], residual=x)
    n2, _, _ = oracle.layernorm_f16(x1, h["ln2_g"], h["ln2_b"], eps)
    f = oracle.gemm_f16(n2, h["w1"], h["b1"], epi="gelu")
    return oracle.gemm_f16(f, h["w2"], h["b2"], residual=x1)


@pytest.mark.parametrize("folded", [False, True])
def test_config2_encoder_block_at_full_size(ctx, folded):
    """``folded``: the block in five launches, its norms folded into the linears that read them (no pass over the rows
    for either), against the same oracle composition that runs them as ops of their own."""
    import torch
    from juliavision_amd import rowstats_
    from juliavision_amd.encoder import EncoderBuffers, FoldedStats, encoder_layer, encoder_layer_folded, fold_layer_norms
    T, d, H, ffn = 1500, 1280, 20, 5120
    h, W = _layer(d, ffn, 1000)
    x = oracle.randn_f16((T, d), 999)
    out = poison(torch.empty((T, d), dtype=torch.float16, device="cuda"))
    if folded:
        dx, st = to_dev(x), FoldedStats(T, d)
        rowstats_(ctx, st.x, dx)
        encoder_layer_folded(ctx, fold_layer_norms(ctx, W), dx, out, EncoderBuffers(T, d, ffn), st, H, 1e-5)
    else:
        encoder_layer(ctx, W, to_dev(x), out, EncoderBuffers(T, d, ffn), H, 1e-5)
    torch.cuda.synchronize()
    want = _oracle_layer(h, x, H, 1e-5)
    assert_parity(to_host(out), want, what="config 2 encoder block")
    # the residual stream alone would already pass a loose gate: what the block ADDED must match too
    assert_parity(to_host(out).astype(np.float32) - x.astype(np.float32), want.astype(np.float32) - x.astype(np.float32),
                  what="config 2 encoder block, update only")


@pytest.mark.parametrize("folded", [False, True])
def test_config3_vit_s14_encoder_at_518(ctx, folded):
    import torch
    from juliavision_amd.encoder import ViTEncoder, ViTWeights
    d, H, ffn, P, S, NL = 384, 6, 1536, 14, 518, 12
    rng = np.random.default_rng(7)
    image = rng.random((1, 3, S, S), dtype=np.float32).astype(np.float16)            # U(0,1)
    patch_w = oracle.randn_f16((d, 3, P, P), 1, 0, 0.02)
    patch_b = oracle.randn_f16((d,), 2, 0, 0.02)
    cls = oracle.randn_f16((1, d), 3, 0, 0.02)
    T = 1 + 37 * 37
    pos = oracle.randn_f16((T, d), 4, 0, 0.02)
    layers = [_layer(d, ffn, 100 + 50 * i) for i in range(NL)]
    norm_g, norm_b = oracle.randn_f16((d,), 5, 1.0, 0.02), oracle.randn_f16((d,), 6, 0.0, 0.02)
    W = ViTWeights(to_dev(patch_w), to_dev(patch_b), to_dev(cls), to_dev(pos), [l[1] for l in layers], to_dev(norm_g), to_dev(norm_b))
    enc = ViTEncoder(W, (S, S), H, ffn, fold_norms=ctx if folded else None)
    assert enc.T == T == 1370
    got = to_host(enc(ctx, to_dev(image)))
    torch.cuda.synchronize()

    emb = oracle.conv2d_f16(image, patch_w, patch_b, (P, P))                          # (1, d, 37, 37)
    tok = np.empty((T, d), dtype=np.float16)
    tok[1:] = oracle.add_f16(np.ascontiguousarray(emb[0].reshape(d, T - 1).T), pos[1:])
    tok[:1] = oracle.add_f16(cls, pos[:1])
    x = tok
    for hl, _ in layers:
        x = _oracle_layer(hl, x, H, 1e-6)
    want, _, _ = oracle.layernorm_f16(x, norm_g, norm_b, 1e-6)
    assert_parity(got, want, what="config 3 ViT-S/14 encoder, 12 layers")
    # the embedding on its own (a fresh run of the first stage)
    assert_parity(to_host(enc.embed(ctx, to_dev(image))), tok, what="config 3 patch embedding + cls + pos")


@pytest.mark.parametrize("layout", ["kf", "fk"])
@pytest.mark.parametrize("B", [1, 4, 8])
def test_config5_decoder_layer_step_at_full_size(ctx, B, layout):
    """One token through a Whisper-decoder-shaped layer at cache position 3 (where the reference records its
    step, plans/whisper-decoder.md:140-142) and at the last slot, 447."""
    import torch
    from juliavision_amd.decode import DecodeBuffers, KVCache, decoder_layer_step
    from test_decode_gpu import _oracle_layer_step, _weights
    d, H, E, ffn, Lmax, Ls = 1280, 20, 64, 5120, 448, 1500
    Wh, Wd = _weights(d, ffn, 500, layout)
    cache = KVCache(1, B, H, E, max_target=Lmax, src_len=Ls)
    ck, cv = oracle.randn_f16((1, B, H, Ls, E), 31), oracle.randn_f16((1, B, H, Ls, E), 32)
    cache.cross_k.copy_(to_dev(ck))
    cache.cross_v.copy_(to_dev(cv))
    buf = DecodeBuffers(B, d, ffn)
    out = torch.empty((B, d), dtype=torch.float16, device="cuda")
    for pos in (3, 447):
        hk, hv = oracle.randn_f16((B, H, Lmax, E), 40 + pos), oracle.randn_f16((B, H, Lmax, E), 41 + pos)
        hk[:, :, pos:] = 0
        hv[:, :, pos:] = 0
        cache.self_k[0].copy_(to_dev(hk))
        cache.self_v[0].copy_(to_dev(hv))
        cache.length.fill_(pos)
        x = oracle.randn_f16((B, d), 60 + pos)
        cache.advance(ctx)
        poison(out)
        decoder_layer_step(ctx, Wd, cache, 0, to_dev(x), out, buf)
        torch.cuda.synchronize()
        length = np.full((B,), pos + 1, dtype=np.int32)
        want = _oracle_layer_step(Wh, x, hk, hv, ck[0], cv[0], length, H, E)
        assert_parity(to_host(out), want, what=f"config 5 decoder layer B{B} {layout} pos {pos}")
        assert_parity(to_host(out).astype(np.float32) - x.astype(np.float32), want.astype(np.float32) - x.astype(np.float32),
                      what=f"config 5 decoder layer B{B} {layout} pos {pos}, update only")
