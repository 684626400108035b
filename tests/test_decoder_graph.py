"""The exported decoder step (tools/export_whisper_decoder.py:90-240) run from its graph: the functional cache
update folded into an in-place write fused with the attention, the position mask into a device-side key count,
the returned cache into an alias of the input; and graphs with symbolic extents bound at load."""
import numpy as np
import pytest

from util import assert_parity, to_dev, to_host


def _decoder_step(layers=2, d=128, heads=2, ffn=256, vocab=100, maxpos=32, seed=0, embed=True, kbias=False):
    """A decoder step written the way the reference's ``DecoderStep`` wrapper is: token + position embedding, the
    ``arange <= cache_position`` mask, per layer a pre-LN self-attention whose new K/V rows go into the cache with
    ``index_copy`` (query scaled by head_dim ** -0.5 ahead of an attention with scale 1), cross-attention over
    precomputed K/V, a GELU MLP; final norm and logits through the tied embedding matrix; the new caches returned
    through ``stack``.  ``embed=False`` drops both ends: hidden state in, hidden state out (one or more bare layers)."""
    import torch
    import torch.nn as nn
    import torch.nn.functional as F

    class Layer(nn.Module):
        def __init__(self):
            super().__init__()
            self.ln1, self.ln2, self.ln3 = nn.LayerNorm(d), nn.LayerNorm(d), nn.LayerNorm(d)
            self.q, self.k, self.v, self.o = nn.Linear(d, d), nn.Linear(d, d, bias=kbias), nn.Linear(d, d), nn.Linear(d, d)
            self.cq, self.co = nn.Linear(d, d), nn.Linear(d, d)
            self.fc1, self.fc2 = nn.Linear(d, ffn), nn.Linear(ffn, d)

    class Step(nn.Module):
        def __init__(self):
            super().__init__()
            if embed:
                self.embed_tokens, self.embed_positions = nn.Embedding(vocab, d), nn.Embedding(maxpos, d)
                self.layer_norm = nn.LayerNorm(d)
            self.layers = nn.ModuleList([Layer() for _ in range(layers)])

        def forward(self, x, self_k, self_v, cross_k, cross_v, cache_position):
            H, hd = heads, d // heads
            B, T = self_k.shape[1], self_k.shape[3]
            scaling = hd ** -0.5
            h = self.embed_tokens(x) + self.embed_positions.weight[cache_position] if embed else x
            idx = torch.arange(T, device=h.device)
            lowest = torch.full((), torch.finfo(h.dtype).min, dtype=h.dtype, device=h.device)
            mask = torch.where(idx <= cache_position, torch.zeros((), dtype=h.dtype, device=h.device), lowest)
            mask = mask.view(1, 1, 1, T).expand(B, H, 1, T)
            heads_of = lambda t: t.view(B, 1, H, hd).transpose(1, 2)
            newk, newv = [], []
            for i, l in enumerate(self.layers):
                r, h = h, l.ln1(h)
                q = heads_of(l.q(h) * scaling)
                K = self_k[i].index_copy(2, cache_position, heads_of(l.k(h)))
                V = self_v[i].index_copy(2, cache_position, heads_of(l.v(h)))
                newk.append(K)
                newv.append(V)
                o = F.scaled_dot_product_attention(q, K, V, attn_mask=mask, scale=1.0)
                h = r + l.o(o.transpose(1, 2).reshape(B, 1, d))
                r, h = h, l.ln2(h)
                o = F.scaled_dot_product_attention(heads_of(l.cq(h) * scaling), cross_k[i], cross_v[i], attn_mask=None, scale=1.0)
                h = r + l.co(o.transpose(1, 2).reshape(B, 1, d))
                r, h = h, l.ln3(h)
                h = r + l.fc2(F.gelu(l.fc1(h)))
            if embed:
                h = F.linear(self.layer_norm(h), self.embed_tokens.weight)
            return h, torch.stack(newk), torch.stack(newv)

    torch.manual_seed(seed)
    return Step().eval().half()


def _args(B=2, layers=2, heads=2, hd=64, T=32, S=40, vocab=100, seed=0, device="cpu"):
    import torch
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: (torch.randn(*s, generator=g) * 0.5).half().to(device)
    return (torch.randint(0, vocab, (B, 1), generator=g).to(device), torch.zeros(layers, B, heads, T, hd).half().to(device),
            torch.zeros(layers, B, heads, T, hd).half().to(device), r(layers, B, heads, S, hd), r(layers, B, heads, S, hd),
            torch.tensor([0]).to(device))


def _export(m, args, mode):
    """composite: as exported; decomposed: core ATen with the fused attention op kept (index_copy -> index_put,
    stack -> cat + view, linear -> addmm); backend: decomposed on the GPU, where attention becomes the accelerator's
    own op -- what the reference's exporter writes (``ep.run_decompositions()`` on its device)."""
    import torch
    ep = torch.export.export(m, args)
    if mode == "decomposed":
        table = torch.export.default_decompositions()
        table.pop(torch.ops.aten.scaled_dot_product_attention.default, None)
        ep = ep.run_decompositions(table)
    elif mode == "backend":
        ep = ep.run_decompositions()
    return ep


@pytest.mark.parametrize("mode", ["composite", "decomposed"])
def test_cache_step_folds_into_in_place_appends(mode):
    from juliavision_amd import graph as G
    m = _decoder_step()
    d = G.convert(_export(m, _args(), mode), "dec")
    aten = [o["aten"] for o in d["ops"]]
    write = "index_copy.default" if mode == "composite" else "index_put.default"
    assert aten.count(write) == 4 and aten.count("where.self") == 1 and aten.count("embedding.default") == 1
    g = G.optimize(G.Graph.load(d))
    left = [o["aten"] for o in g.ops]
    # the writes, the mask arithmetic and the stacking of the returned cache are gone
    for gone in (write, "where.self", "le.Tensor", "arange.default", "arange.start_step", "full.default", "zeros.default",
                 "stack.default", "cat.default", "index.Tensor", "add.Tensor"):
        assert gone not in left, (gone, g.notes)
    assert left.count("sdpa_append") == 2 and left.count("kv_len_from_position") == 1 and left.count("embedding.default") == 1
    assert left[0] == "kv_len_from_position"
    app = [o for o in g.ops if o["aten"] == "sdpa_append"]
    for layer, o in enumerate(app):
        q, ck, cv, kn, vn, n = o["in"]
        assert g.root(ck) == "self_k" and g.root(cv) == "self_v" and g.buffers[ck]["attrs"]["arg2"] == layer
        assert g.buffers[n]["dtype"] == "int32" and g.buffers[n]["shape"] == [2] and "masked" not in o["attrs"]
    # the returned caches are the inputs
    assert [g.root(o) for o in g.outputs[1:]] == ["self_k", "self_v"]
    # the cross-attention stays an ordinary fused attention; token + position embedding is one gather
    assert sum(a in G.SDPA_OPS for a in left) == 2
    emb = next(o for o in g.ops if o["aten"] == "embedding.default")
    assert len(emb["in"]) == 4 and emb["in"][1] == "x" and emb["in"][3] == "cache_position"
    # q, k and v read one norm: a single product over their weights end to end, the norm as its prologue; every other
    # norm sits in front of one linear and becomes that linear's prologue -- no norm launch is left, 8 launches a layer
    groups = [o for o in g.ops if o["aten"] == "linear_group"]
    assert len(groups) == 2 and all(len(o["attrs"]["members"]) == 3 and o["attrs"]["ln_in"] for o in groups), g.notes
    assert groups[0]["attrs"]["ln_in_gamma"].endswith("layers_0_ln1_weight")
    assert not any("layer_norm" in a for a in left) and len(left) == 3 + 2 * 8


def test_cache_write_that_someone_else_reads_is_left_functional():
    """If the graph also returns one layer's updated plane on its own -- or reads the old plane after the write -- the
    update must stay a copy: nothing is folded, and the executor then names the op it has no kernel for."""
    import torch
    from juliavision_amd import graph as G
    m = _decoder_step(layers=1, embed=False)

    class AlsoOld(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.m = m

        def forward(self, x, sk, sv, ck, cv, pos):
            h, nk, nv = self.m(x, sk, sv, ck, cv, pos)
            return h, nk, nv, sk[0].sum(-1)            # reads the plane the fold would overwrite

    a = _args(layers=1)
    x = torch.randn(2, 1, 128).half()
    g = G.optimize(G.Graph.load(G.convert(torch.export.export(AlsoOld().eval(), (x,) + a[1:]), "dec")))
    left = [o["aten"] for o in g.ops]
    assert "sdpa_append" not in left and left.count("index_copy.default") == 2, g.notes


def test_a_mask_that_is_not_the_position_mask_stays_an_operand():
    import torch
    import torch.nn.functional as F
    from juliavision_amd import graph as G

    class Step(torch.nn.Module):
        def forward(self, q, k_new, v_new, sk, sv, pos, mask):
            K, V = sk.index_copy(2, pos, k_new), sv.index_copy(2, pos, v_new)
            return F.scaled_dot_product_attention(q, K, V, attn_mask=mask), K, V

    B, H, T, E = 2, 2, 16, 64
    z = lambda *s: torch.zeros(*s).half()
    ep = torch.export.export(Step(), (z(B, H, 1, E), z(B, H, 1, E), z(B, H, 1, E), z(B, H, T, E), z(B, H, T, E), torch.tensor([3]), z(B, 1, 1, T)))
    g = G.optimize(G.Graph.load(G.convert(ep, "one")))
    o = next(o for o in g.ops if o["aten"] == "sdpa_append")
    assert o["attrs"].get("masked") and o["in"][6] == "mask" and o["in"][1:3] == ["sk", "sv"]
    assert [g.root(x) for x in g.outputs[1:]] == ["sk", "sv"]


def test_symbolic_extents_are_bound_at_load():
    """A graph exported with a dynamic token count keeps its extents as expressions; ``Graph.load`` binds them
    (``evalshape``, graph.jl:150-167) and the bound graph is an ordinary static one."""
    import torch
    from juliavision_amd import graph as G

    class M(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.ln, self.fc1, self.fc2 = torch.nn.LayerNorm(64), torch.nn.Linear(64, 128), torch.nn.Linear(128, 64)

        def forward(self, x):
            B, T, D = x.shape
            y = self.fc2(torch.nn.functional.gelu(self.fc1(self.ln(x))))
            return (x + y).view(B * T, D)

    m = M().eval().half()
    T = torch.export.Dim("T", min=2, max=512)
    ep = torch.export.export(m, (torch.randn(2, 24, 64).half(),), dynamic_shapes={"x": {1: T}}).run_decompositions()
    d = G.convert(ep, "dyn")
    assert len(d["symbols"]) == 1
    s = d["symbols"][0]
    assert next(b for b in d["buffers"] if b["id"] == d["inputs"][0])["shape"] == [2, s, 64]
    with pytest.raises(ValueError, match="need values"):
        G.Graph.load(d)
    for n in (24, 100):
        g = G.Graph.load(d, dims={s: n})
        assert g.buffers[g.inputs[0]]["shape"] == [2, n, 64] and g.buffers[g.outputs[0]]["shape"] == [2 * n, 64]
        for b in g.buffers.values():                     # nothing symbolic is left anywhere
            assert all(isinstance(x, int) for x in b.get("shape", []))
            if b["kind"] == "view":
                assert all(isinstance(x, int) for v in b["attrs"].values() if isinstance(v, list) for x in v), b
        g = G.optimize(g)
        assert [o["aten"] for o in g.ops].count("gelu.default") == 0


def test_extent_expressions():
    from juliavision_amd.graph import UnsupportedOp, evalexpr
    dims = {"h": 10, "w": 4, "s0": 7}
    assert evalexpr("h*w", dims) == 40 and evalexpr("((s0 + 1)//2)", dims) == 4 and evalexpr("2*h + 1 - w", dims) == 17
    assert evalexpr("Mod(h, 3)", dims) == 1 and evalexpr("Max(h, w) + Min(h, w)", dims) == 14 and evalexpr("w**2", dims) == 16
    assert evalexpr("ceiling(h/3)", dims) == 4 and evalexpr("floor(h/3)", dims) == 3 and evalexpr("h/3", dims) == 3
    assert evalexpr("-(-h//3)", dims) == 4 and evalexpr(12, dims) == 12
    with pytest.raises(KeyError):
        evalexpr("h*c", dims)
    for bad in ("__import__('os')", "h.real", "[h]", "h if w else 1", "print(h)"):
        with pytest.raises(UnsupportedOp):
            evalexpr(bad, dims)


# ----------------------------------------------------------------------------- on the GPU

def _functional_steps(m, args, tokens, positions):
    """The module itself in fp32 on the CPU, token by token, feeding the returned cache back in."""
    import torch
    ids, sk, sv, ck, cv, _ = args
    m32 = _clone_fp32(m)
    sk, sv, ck, cv = sk.float(), sv.float(), ck.float(), cv.float()
    outs = []
    with torch.no_grad():
        for tok, p in zip(tokens, positions):
            y, sk, sv = m32(tok, sk, sv, ck, cv, torch.tensor([p]))
            outs.append(y.numpy())
    return outs, sk.numpy(), sv.numpy()


def _clone_fp32(m):
    import copy
    return copy.deepcopy(m).float()


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["composite", "decomposed", "backend"])
def test_exported_decoder_step_runs_in_place(ctx, mode):
    import torch
    from juliavision_amd import graph as G
    m = _decoder_step(seed=3)
    args = _args(seed=4)
    if mode == "backend":
        ep = _export(m.cuda(), tuple(a.cuda() for a in args), mode)
        m = m.cpu()
    else:
        ep = _export(m, args, mode)
    g = G.optimize(G.Graph.load(G.convert(ep, "dec")))
    assert [o["aten"] for o in g.ops].count("sdpa_append") == 2, g.notes
    run = G.Executor(g, m.state_dict(), ctx)
    gen = torch.Generator().manual_seed(5)
    tokens = [torch.randint(0, 100, (2, 1), generator=gen) for _ in range(6)]
    want, want_k, want_v = _functional_steps(m, args, tokens, range(6))
    ids, sk, sv, ck, cv, pos = (a.cuda() for a in args)
    for t, tok in enumerate(tokens):
        ids.copy_(tok)
        pos.fill_(t)
        logits, nk, nv = run(ids, sk, sv, ck, cv, pos)
        torch.cuda.synchronize()
        assert nk.data_ptr() == sk.data_ptr() and nv.data_ptr() == sv.data_ptr()      # the caller's cache, updated
        assert_parity(to_host(logits.float()), want[t], what=f"{mode} logits at position {t}")
    assert_parity(to_host(sk.float()), want_k, what="self_k after six steps")
    assert_parity(to_host(sv.float()), want_v, what="self_v after six steps")
    assert not to_host(sk[:, :, :, 6:]).any()                                       # slots past the position untouched


@pytest.mark.gpu
def test_exported_decoder_step_replays_as_one_graph(ctx):
    """Captured once; each replay follows the token and position tensors' contents, appends in place, and equals the
    eager run of the same step on a twin cache bit for bit (eager work and synchronisations between replays)."""
    import torch
    from juliavision_amd import graph as G
    m = _decoder_step(seed=6)
    args = _args(seed=7)
    g = G.optimize(G.Graph.load(G.convert(_export(m, args, "decomposed"), "dec")))
    run, twin = G.Executor(g, m.state_dict(), ctx), G.Executor(g, m.state_dict(), ctx)
    ids, sk, sv, ck, cv, pos = (a.cuda() for a in args)
    sk2, sv2 = sk.clone(), sv.clone()
    pos.fill_(31)                                        # capture at the last slot; the cache is restored below
    replay, outs = run.replayable(ids, sk, sv, ck, cv, pos)
    sk.zero_()
    sv.zero_()
    gen = torch.Generator().manual_seed(8)
    for t in range(5):
        ids.copy_(torch.randint(0, 100, (2, 1), generator=gen))
        pos.fill_(t)
        replay()
        torch.cuda.synchronize()
        got = outs[0].clone()
        want, _, _ = twin(ids, sk2, sv2, ck, cv, pos)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay at position {t} differs from the eager step"
        assert torch.equal(sk, sk2) and torch.equal(sv, sv2)


@pytest.mark.gpu
@pytest.mark.parametrize("B", [1, 4])
def test_exported_decoder_layer_matches_the_oracle_layer_step(ctx, B):
    """One bare decoder layer, exported, against the CPU composition of the oracle's kernels that the hand-written
    layer step is tested with (same weights, same ragged-free history): the q scaling of 0.125 is exact in fp16, so
    the two describe the same arithmetic."""
    import torch
    import oracle
    from juliavision_amd import graph as G
    from test_decode_gpu import _oracle_layer_step
    d, H, E, ffn, T, S = 256, 4, 64, 512, 12, 70
    m = _decoder_step(layers=1, d=d, heads=H, ffn=ffn, embed=False, kbias=True, seed=1)
    l = m.layers[0]
    Wh = {}
    # the oracle's packed [K][F] weights from the module's [F][K] ones; the query scaling lives in the oracle's attention
    Wh["wqkv"] = np.concatenate([to_host_np(x.weight).T for x in (l.q, l.k, l.v)], axis=1)
    Wh["bqkv"] = np.concatenate([to_host_np(x.bias) for x in (l.q, l.k, l.v)])
    for name, lin in (("wo", l.o), ("wq_c", l.cq), ("wo_c", l.co), ("w1", l.fc1), ("w2", l.fc2)):
        Wh[name] = np.ascontiguousarray(to_host_np(lin.weight).T)
    for name, lin in (("bo", l.o), ("bq_c", l.cq), ("bo_c", l.co), ("b1", l.fc1), ("b2", l.fc2)):
        Wh[name] = to_host_np(lin.bias)
    for name, ln in (("ln1", l.ln1), ("ln2", l.ln2), ("ln3", l.ln3)):
        Wh[name + "_g"], Wh[name + "_b"] = to_host_np(ln.weight), to_host_np(ln.bias)
    start = 5
    hk, hv = np.zeros((B, H, T, E), np.float16), np.zeros((B, H, T, E), np.float16)
    hk[:, :, :start] = oracle.randn_f16((B, H, start, E), 40)
    hv[:, :, :start] = oracle.randn_f16((B, H, start, E), 50)
    ck, cv = oracle.randn_f16((1, B, H, S, E), 31), oracle.randn_f16((1, B, H, S, E), 32)
    x0 = torch.zeros(B, 1, d).half()
    ex = (x0, torch.zeros(1, B, H, T, E).half(), torch.zeros(1, B, H, T, E).half(), torch.from_numpy(ck), torch.from_numpy(cv), torch.tensor([0]))
    g = G.optimize(G.Graph.load(G.convert(_export(m, ex, "decomposed"), "layer")))
    run = G.Executor(g, m.state_dict(), ctx)
    sk, sv = to_dev(hk[None]), to_dev(hv[None])
    for step in range(3):
        x = oracle.randn_f16((B, d), 60 + step)
        p = start + step
        out, nk, nv = run(to_dev(x).view(B, 1, d), sk, sv, to_dev(ck), to_dev(cv), torch.tensor([p]).cuda())
        torch.cuda.synchronize()
        want = _oracle_layer_step(Wh, x, hk, hv, ck[0], cv[0], np.full((B,), p + 1), H, E)
        assert_parity(to_host(out).reshape(B, d), want, what=f"exported layer B{B} step {step}")
        assert_parity(to_host(sk[0]), hk, what=f"self_k after step {step}")
        assert_parity(to_host(sv[0]), hv, what=f"self_v after step {step}")


def to_host_np(t):
    return t.detach().cpu().numpy()


@pytest.mark.gpu
def test_symbolic_graph_runs_at_two_bindings(ctx):
    import torch
    from juliavision_amd import graph as G

    class M(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.ln, self.fc1, self.fc2 = torch.nn.LayerNorm(128), torch.nn.Linear(128, 256), torch.nn.Linear(256, 128)

        def forward(self, x):
            B, T, D = x.shape
            return (x + self.fc2(torch.nn.functional.gelu(self.fc1(self.ln(x))))).view(B * T, D)

    torch.manual_seed(2)
    m = M().eval().half()
    T = torch.export.Dim("T", min=2, max=512)
    d = G.convert(torch.export.export(m, (torch.randn(2, 24, 128).half(),), dynamic_shapes={"x": {1: T}}).run_decompositions(), "dyn")
    for n in (24, 70):
        run = G.Executor(G.optimize(G.Graph.load(d, dims={d["symbols"][0]: n})), m.state_dict(), ctx)
        x = torch.randn(2, n, 128).half()
        with torch.no_grad():
            want = _clone_fp32(m)(x.float()).numpy()
        got = run(x.cuda())
        torch.cuda.synchronize()
        assert got.shape == (2 * n, 128)
        assert_parity(to_host(got.float()), want, what=f"dynamic token count bound to {n}")


@pytest.mark.gpu
def test_embedding_gathers_rows_bit_exactly(ctx):
    import torch
    from juliavision_amd import kernels as K
    g = torch.Generator().manual_seed(0)
    for D in (128, 100):                                   # 16-byte chunks, and the element path
        tab, tab2 = torch.randn(50, D, generator=g).half().cuda(), torch.randn(9, D, generator=g).half().cuda()
        ids = torch.randint(0, 50, (3, 4), generator=g).cuda()
        out = torch.full((3, 4, D), float("nan"), dtype=torch.float16, device="cuda")
        K.embedding_(ctx, out, tab, ids)
        assert torch.equal(out, tab[ids])
        one = torch.tensor([7]).cuda()
        K.embedding_(ctx, out, tab, ids, tab2, one)
        assert torch.equal(out, tab[ids] + tab2[one])       # fp16 add of two fp16 values: one rounding either way
        per = torch.randint(0, 9, (12,), generator=g).cuda()
        K.embedding_(ctx, out, tab, ids, tab2, per)
        assert torch.equal(out, tab[ids] + tab2[per].view(3, 4, D))
        ids[0, 0] = 50                                      # outside the table: a row of zeros, nothing read
        K.embedding_(ctx, out, tab, ids)
        assert not out[0, 0].any() and torch.equal(out[1:], tab[ids[1:]])


@pytest.mark.gpu
def test_full_cache_is_left_alone_and_says_so(ctx):
    """A step past the capacity stores nothing, attends over what is stored and leaves length = capacity + 1 behind."""
    import torch
    from juliavision_amd import kernels as K
    from juliavision_amd.decode import KVCache
    B, H, E, Lmax = 2, 2, 64, 8
    cache = KVCache(1, B, H, E, max_target=Lmax, src_len=1)
    g = torch.Generator().manual_seed(1)
    cache.self_k.copy_(torch.randn(1, B, H, Lmax, E, generator=g).half())
    cache.self_v.copy_(torch.randn(1, B, H, Lmax, E, generator=g).half())
    cache.length.copy_(torch.tensor([Lmax, 3], dtype=torch.int32))
    before_k, before_v = cache.self_k.clone(), cache.self_v.clone()
    q, kn, vn = (torch.randn(B, H, 1, E, generator=g).half().cuda() for _ in range(3))
    assert not cache.overflowed()
    cache.advance(ctx)
    out = torch.empty(B, H, 1, E, dtype=torch.float16, device="cuda")
    K.sdpa_append(ctx, q, cache.self_k[0], cache.self_v[0], kn, vn, cache.length, out=out)
    torch.cuda.synchronize()
    assert to_host(cache.length).tolist() == [Lmax + 1, 4] and cache.overflowed()
    assert torch.equal(cache.self_k[0, 0], before_k[0, 0]) and torch.equal(cache.self_v[0, 0], before_v[0, 0])     # row 0: full, untouched
    assert torch.equal(cache.self_k[0, 1, :, 3], kn[1, :, 0]) and torch.equal(cache.self_k[0, 1, :, :3], before_k[0, 1, :, :3])
    want0 = torch.nn.functional.scaled_dot_product_attention(q[:1].float(), before_k[0, :1].float(), before_v[0, :1].float())
    assert_parity(to_host(out[:1].float()), to_host(want0), what="attention over the full cache, new row not stored")
    # the two-call form treats the mark the same way
    cache.append(ctx, 0, kn, vn)
    torch.cuda.synchronize()
    assert torch.equal(cache.self_k[0, 0], before_k[0, 0])
