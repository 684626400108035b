"""Seeded random shapes through the public entry points against the oracle: whatever route the planners pick for a
shape (fused, key halves, short chains, split keys, rows; tiled, split-K, decode-sized, scalar GEMM; 1x1, implicit,
im2col convolution in both output forms), the result is the oracle's.  Every case prints itself before it runs."""
import random

import numpy as np
import pytest

import oracle
from util import assert_parity, poison, to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [7, 23])
def test_attention_random_shapes(ctx, seed):
    import torch
    import juliavision_amd as jv
    rnd = random.Random(seed)
    for it in range(70):
        B, H = rnd.choice([1, 1, 2, 3]), rnd.choice([1, 2, 3, 6, 8, 12, 20])
        E = rnd.choice([64, 64, 64, 48, 32, 72, 80, 96, 128, 16])
        Lq, Lk = rnd.choice([1, 1, 2, 7, rnd.randint(8, 700), rnd.randint(64, 1500)]), rnd.randint(1, 2300)
        if B * H * Lq * Lk > 4.0e7:
            Lk = max(1, int(4.0e7 / (B * H * Lq)))
        mask = rnd.choice([None, None, None, "f16", "f32", "row"])
        use_len = mask is None and rnd.random() < 0.4
        what = f"sdpa seed{seed} #{it} B{B} H{H} Lq{Lq} Lk{Lk} E{E} mask={mask} kv_len={use_len}"
        print(what, flush=True)
        q, k, v = oracle.randn_f16((B, H, Lq, E), it, 0, 1.5), oracle.randn_f16((B, H, Lk, E), it + 1000), oracle.randn_f16((B, H, Lk, E), it + 2000)
        lens = np.array([rnd.randint(0, Lk) for _ in range(B)], dtype=np.int32) if use_len else None
        bias = {None: None, "f16": lambda: oracle.randn_f16((B, H, Lq, Lk), it + 3000, 0, 2.0),
                "f32": lambda: oracle.randn_f32((B, 1, Lq, Lk), it + 3000, 0, 2.0),
                "row": lambda: oracle.randn_f16((1, 1, 1, Lk), it + 3000, 0, 2.0)}[mask]
        bias = None if bias is None else bias()
        out = poison(torch.empty((B, H, Lq, E), dtype=torch.float16, device="cuda"))
        ctx.ws.reset()
        jv.sdpa(ctx, to_dev(q), to_dev(k), to_dev(v), None if bias is None else to_dev(bias), None, out=out,
                kv_len=None if lens is None else torch.from_numpy(lens).cuda())
        torch.cuda.synchronize()
        assert_parity(to_host(out), oracle.sdpa_threepass_f16(q, k, v, bias, kv_len=lens), what=what)


@pytest.mark.parametrize("seed", [5])
def test_attention_random_key_masks(ctx, seed):
    """Masks that are the same for every query -- (1,1,1,Lk), (B,1,1,Lk), (B,H,1,Lk), (1,H,1,Lk); values, or 0 / -inf holes --
    over random extents on both sides of every form the fused kernel has and of the 4096-key limit of the LDS copy."""
    import torch
    import juliavision_amd as jv
    rnd = random.Random(seed)
    for it in range(60):
        B, H = rnd.choice([1, 2, 3, 8]), rnd.choice([1, 2, 6, 16, 20, 40])
        E = rnd.choice([64, 64, 64, 32, 72, 96, 128])
        Lq, Lk = rnd.choice([64, rnd.randint(64, 400), rnd.randint(64, 1500)]), rnd.choice([rnd.randint(1, 2300), rnd.randint(3900, 4300)])
        if B * H * Lq * Lk > 6.0e7:
            H = max(1, int(6.0e7 / (B * Lq * Lk)))
        shape = rnd.choice([(1, 1, 1, Lk), (B, 1, 1, Lk), (B, H, 1, Lk), (1, H, 1, Lk)])
        holes = rnd.random() < 0.5
        what = f"sdpa key mask seed{seed} #{it} B{B} H{H} Lq{Lq} Lk{Lk} E{E} mask{shape} holes={holes}"
        print(what, flush=True)
        q, k, v = oracle.randn_f16((B, H, Lq, E), it, 0, 1.5), oracle.randn_f16((B, H, Lk, E), it + 1000), oracle.randn_f16((B, H, Lk, E), it + 2000)
        if holes:
            gen = np.random.default_rng(seed * 1000 + it)
            bias = np.where(gen.random(shape) < 0.4, -np.inf, 0.0).astype(np.float16)
            bias[..., gen.integers(0, Lk)] = 0.0                     # a key stays in every row
        else:
            bias = oracle.randn_f16(shape, it + 3000, 0, 2.0)
        out = poison(torch.empty((B, H, Lq, E), dtype=torch.float16, device="cuda"))
        ctx.ws.reset()
        jv.sdpa(ctx, to_dev(q), to_dev(k), to_dev(v), to_dev(bias), None, out=out)
        torch.cuda.synchronize()
        assert_parity(to_host(out), oracle.sdpa_threepass_f16(q, k, v, bias), what=what)


@pytest.mark.parametrize("seed", [7, 23])
def test_gemm_random_shapes(ctx, seed):
    import torch
    import juliavision_amd as jv
    rnd = random.Random(seed)
    for it in range(50):
        T = rnd.choice([1, 3, 8, 9, 33, rnd.randint(10, 400), rnd.randint(100, 1600)])
        K, F = rnd.choice([8, 24, 64, 128, 192, 384, 520, 1280, 1536, 2048]), rnd.choice([8, 40, 64, 264, 384, 1000, 1280, 1536])
        layout, epi = rnd.choice(["kf", "fk"]), rnd.choice(["none", "gelu", "relu"])
        res, norm = rnd.random() < 0.5, rnd.random() < 0.4
        what = f"gemm seed{seed} #{it} T{T} K{K} F{F} {layout} {epi} residual={res} norm={norm}"
        print(what, flush=True)
        X, W = oracle.randn_f16((T, K), it, 0, 1.0 / np.sqrt(K)), oracle.randn_f16((K, F), it + 500, 0, 1.0)
        b, R = oracle.randn_f16((F,), it + 600, 0, 0.1), (oracle.randn_f16((T, F), it + 700) if res else None)
        g, be = oracle.randn_f16((F,), it + 800, 1.0, 0.2), oracle.randn_f16((F,), it + 900, 0, 0.2)
        Wd = to_dev(W) if layout == "kf" else to_dev(np.ascontiguousarray(W.T)).t()
        y, h = (poison(torch.empty((T, F), dtype=torch.float16, device="cuda")) for _ in range(2))
        want = oracle.gemm_f16(X, W, b, epi=epi, residual=R)
        ctx.ws.reset()
        if norm:
            jv.matmul_ln_(ctx, y, h, Wd, to_dev(X), to_dev(g), to_dev(be), 1e-6, to_dev(b), epi=epi, residual=None if R is None else to_dev(R))
        else:
            jv.matmul_(ctx, y, Wd, to_dev(X), to_dev(b), epi=epi, residual=None if R is None else to_dev(R))
        torch.cuda.synchronize()
        assert_parity(to_host(y), want, what=what)
        if norm:
            # the norm of the device's own rows: a last-bit difference in y is amplified by 1 / sigma and is not the norm's error
            assert_parity(to_host(h), oracle.layernorm_f16(to_host(y), g, be, 1e-6)[0], what=what + " (norm)")


@pytest.mark.parametrize("seed", [7, 23])
def test_convolution_random_shapes(ctx, seed):
    import torch
    import juliavision_amd as jv
    rnd = random.Random(seed)
    for it in range(40):
        N, Cin, Cout = rnd.choice([1, 1, 2]), rnd.choice([1, 3, 5, 16, 32, 64]), rnd.choice([8, 24, 64, 144])
        KH = rnd.choice([1, 2, 3, 5, 8])
        KW = rnd.choice([KH, KH, 1, 3])
        s, p = rnd.choice([1, 1, 2, KH]), rnd.choice([0, 0, 1, 2])
        Hi, Wi = rnd.randint(max(KH, 4), 40), rnd.randint(max(KW, 4), 40)
        OH, OW = oracle.convsize(Hi, KH, s, p, 1), oracle.convsize(Wi, KW, s, p, 1)
        tokens = rnd.random() < 0.5
        what = f"conv seed{seed} #{it} N{N} Cin{Cin} {Hi}x{Wi} Cout{Cout} k{KH}x{KW} s{s} p{p} tokens={tokens}"
        print(what, flush=True)
        x, w = oracle.randn_f16((N, Cin, Hi, Wi), it), oracle.randn_f16((Cout, Cin, KH, KW), it + 100, 0, 0.1)
        b = oracle.randn_f16((Cout,), it + 200, 0, 0.5)
        want = oracle.conv2d_f16(x, w, b, (s, s), (p, p), (1, 1), 1, False)
        ctx.ws.reset()
        if tokens:
            r = oracle.randn_f16((OH * OW, Cout), it + 300)
            out = poison(torch.empty((N, OH * OW, Cout), dtype=torch.float16, device="cuda"))
            jv.convolution_tokens_(ctx, out, to_dev(x), to_dev(w), to_dev(b), (s, s), (p, p), (1, 1), residual=to_dev(r))
            want = (want.reshape(N, Cout, OH * OW).transpose(0, 2, 1).astype(np.float32) + r.astype(np.float32)).astype(np.float16)
        else:
            out = poison(torch.empty(want.shape, dtype=torch.float16, device="cuda"))
            jv.convolution_(ctx, out, to_dev(x), to_dev(w), to_dev(b), (s, s), (p, p), (1, 1), 1)
        torch.cuda.synchronize()
        assert_parity(to_host(out), want, what=what)
