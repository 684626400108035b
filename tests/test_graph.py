"""The exported-graph loader/executor: schema conversion and rewrites on the CPU, execution on the GPU against
the same module evaluated by torch in fp32 (the module's own arithmetic, independent of this library)."""
import json

import numpy as np
import pytest

from util import assert_parity


def _block(d=128, heads=2, ffn=256, seed=0):
    import torch
    import torch.nn as nn
    import torch.nn.functional as F

    class Block(nn.Module):
        """A pre-LN encoder block written the way the exported models are: separate q/k/v linears (k without bias,
        as in Whisper), SDPA on (B, H, T, E) views, GELU MLP, two residual adds."""

        def __init__(self):
            super().__init__()
            self.h = heads
            self.ln1, self.ln2 = nn.LayerNorm(d), nn.LayerNorm(d)
            self.q, self.k, self.v, self.o = nn.Linear(d, d), nn.Linear(d, d, bias=False), nn.Linear(d, d), nn.Linear(d, d)
            self.fc1, self.fc2 = nn.Linear(d, ffn), nn.Linear(ffn, d)

        def forward(self, x):
            B, T, D = x.shape
            y = self.ln1(x)
            sp = lambda t: t.view(B, T, self.h, D // self.h).transpose(1, 2)
            a = F.scaled_dot_product_attention(sp(self.q(y)), sp(self.k(y)), sp(self.v(y)))
            x = x + self.o(a.transpose(1, 2).reshape(B, T, D))
            return x + self.fc2(F.gelu(self.fc1(self.ln2(x))))

    torch.manual_seed(seed)
    m = Block().eval()
    with torch.no_grad():
        for p in m.parameters():
            if p.dim() == 1:
                p.copy_(torch.randn_like(p) * 0.1 + (1.0 if p is m.ln1.weight or p is m.ln2.weight else 0.0))
    return m.half()


def _export(m, T=70, d=128):
    import torch
    x = torch.randn(1, T, d).half()
    return torch.export.export(m, (x,)), x


def test_convert_writes_the_reference_schema():
    from juliavision_amd import graph as G
    m = _block()
    ep, _ = _export(m)
    d = G.convert(ep, "block")
    json.loads(json.dumps(d))                                         # plain JSON
    assert set(d) >= {"name", "symbols", "inputs", "outputs", "buffers", "ops", "fusion_groups", "barriers"}
    kinds = {b["id"]: b["kind"] for b in d["buffers"]}
    assert d["inputs"] == ["x"] and kinds["x"] == "external" and kinds[d["outputs"][0]] == "external"
    weights = [b for b in d["buffers"] if b["kind"] == "weight"]
    assert {b["key"] for b in weights} == set(m.state_dict())
    assert kinds["view"] == "view" and kinds["transpose"] == "view"
    aten = [o["aten"] for o in d["ops"]]
    assert aten.count("linear.default") == 6 and aten.count("scaled_dot_product_attention.default") == 1
    assert aten.count("layer_norm.default") == 2 and aten.count("gelu.default") == 1 and aten.count("add.Tensor") == 2
    lin = next(o for o in d["ops"] if o["id"] == "linear")
    assert lin["in"] == ["layer_norm", "p_q_weight", "p_q_bias"] and lin["out"] == "linear"
    tr = next(b for b in d["buffers"] if b["id"] == "transpose")
    assert tr["of"] == "view" and tr["op"] == "transpose.int" and tr["attrs"]["arg1"] == 1 and tr["attrs"]["arg2"] == 2
    live = next(b for b in d["buffers"] if b["id"] == "layer_norm")["live"]
    assert live[0] == 0 and live[1] == aten.index("scaled_dot_product_attention.default") - 1   # last read by the v projection


def test_rewrites_fold_activation_residuals_and_attention_layout():
    from juliavision_amd import graph as G
    ep, _ = _export(_block())
    g = G.optimize(G.Graph.load(G.convert(ep, "block")))
    aten = [o["aten"] for o in g.ops]
    assert "gelu.default" not in aten and "add.Tensor" not in aten
    fc1 = g.op("linear_4")
    assert fc1["attrs"]["epilogue"] == "gelu" and g.buffers["gelu"]["kind"] == "view" and g.buffers["gelu"]["of"] == "linear_4"
    assert g.op("linear_3")["attrs"]["residual"] == "$x" and g.op("linear_5")["attrs"]["residual"] == "$add"
    assert g.op("scaled_dot_product_attention")["attrs"]["token_major"] is True
    assert len(g.ops) == 6                                              # row statistics of x, q/k/v as one group, attention, 3 linears
    grp = next(o for o in g.ops if o["aten"] == "linear_group")
    assert [m["out"] for m in grp["attrs"]["members"]] == ["linear", "linear_1", "linear_2"]
    assert g.root("add_1") == "linear_5" and len(g.notes) == 7
    # 70 rows are enough for the tiled GEMMs: neither norm has a pass of its own.  The first reads the graph's input, whose
    # row statistics one small op computes where the norm stood; q, k and v run on the raw rows as planes of one launch
    assert g.op("layer_norm") is None and g.op("layer_norm_1") is None
    assert [o["aten"] for o in g.ops][:2] == ["rowstats", "linear_group"] and g.ops[0]["in"] == ["x"]
    assert grp["attrs"]["lnf"] == g.ops[0]["out"] and grp["attrs"]["lnf_gamma"] == "p_ln1_weight" and grp["attrs"]["lnf_beta"] == "p_ln1_bias"
    assert g.buffers[g.ops[0]["out"]]["shape"] == [4, 70, 2] and g.buffers["layer_norm"]["of"] == "x"
    # the second reads the residual stream the out-projection writes: that GEMM leaves the statistics, fc1 takes them
    proj = g.op("linear_3")
    assert "ln_out" not in proj["attrs"] and fc1["attrs"]["lnf"] == proj["attrs"]["stats_out"] and fc1["attrs"]["lnf_eps"] == 1e-5
    assert fc1["attrs"]["lnf_gamma"] == "p_ln2_weight" and g.buffers["layer_norm_1"]["of"] == "add"
    # fewer rows than a tile is worth: the norms stay, the second as the out-projection's second result
    ep40, _ = _export(_block(), T=40)
    g40 = G.optimize(G.Graph.load(G.convert(ep40, "block")))
    proj = g40.op("linear_3")
    assert proj["attrs"]["ln_out"] == "layer_norm_1" and proj["attrs"]["ln_gamma"] == "p_ln2_weight" and proj["attrs"]["ln_eps"] == 1e-5
    assert g40.op("layer_norm_1") is None and g40.op("layer_norm") is not None and not any("lnf" in o["attrs"] for o in g40.ops)
    # an activation that something else also reads must stay where it is
    d = G.convert(ep, "block")
    d["outputs"].append("linear_4")
    g2 = G.fold_activations(G.Graph.load(d))
    assert any(o["aten"] == "gelu.default" for o in g2.ops)


def test_unsupported_op_is_named():
    import torch
    from juliavision_amd import graph as G

    class M(torch.nn.Module):
        def forward(self, x):
            return torch.tanh(x)

    ep = torch.export.export(M(), (torch.randn(2, 8).half(),))
    g = G.Graph.load(G.convert(ep, "m"))
    assert [o["aten"] for o in g.ops] == ["tanh.default"]
    assert "tanh.default" not in G.Executor.HANDLERS


@pytest.mark.gpu
@pytest.mark.parametrize("fold", [True, False])
def test_exported_block_runs_on_the_kernels(ctx, fold):
    import torch
    from juliavision_amd import graph as G
    m = _block(seed=3)
    ep, x = _export(m)
    g = G.Graph.load(G.convert(ep, "block"))
    if fold:
        g = G.optimize(g)
    else:
        g = G.fold_sdpa_transpose(G.fold_activations(g))          # residual adds stay separate ops
        assert sum(o["aten"] == "add.Tensor" for o in g.ops) == 2
    run = G.Executor(g, m.state_dict(), ctx)
    with torch.no_grad():
        want = m.float()(x.float()).numpy()
    got = run(x.cuda())
    torch.cuda.synchronize()
    assert_parity(got.float().cpu().numpy(), want, what=f"exported block fold={fold}")
    x2 = torch.randn_like(x)                                       # same executor, new input: nothing is cached
    with torch.no_grad():
        want2 = m(x2.float()).numpy()
    assert_parity(run(x2.cuda()).float().cpu().numpy(), want2, what="second call")


def _mlp(d=256, ffn=512, seed=0):
    import torch
    import torch.nn as nn
    import torch.nn.functional as F

    class MLP(nn.Module):
        """The feed-forward half of a pre-LN decoder layer, as a decoder step sees it: a handful of token rows."""

        def __init__(self):
            super().__init__()
            self.ln, self.fc1, self.fc2 = nn.LayerNorm(d), nn.Linear(d, ffn), nn.Linear(ffn, d)

        def forward(self, x):
            return x + self.fc2(F.gelu(self.fc1(self.ln(x))))

    torch.manual_seed(seed)
    return MLP().eval().half()


def test_decode_sized_norm_becomes_the_prologue_of_the_linear_that_reads_it():
    import torch
    from juliavision_amd import graph as G
    m = _mlp()
    for rows, folded in ((4, True), (40, False), (300, None)):
        ep = torch.export.export(m, (torch.randn(1, rows, 256).half(),))
        g = G.optimize(G.Graph.load(G.convert(ep, "mlp")))
        fc1 = g.op("linear")
        if folded:      # norm -> fc1's prologue, gelu -> its epilogue, add -> fc2's store: two launches
            assert [o["aten"] for o in g.ops] == ["linear.default", "linear.default"], g.notes
            assert fc1["attrs"]["ln_in"] is True and fc1["attrs"]["ln_in_gamma"] == "p_ln_weight" and fc1["attrs"]["epilogue"] == "gelu"
            assert g.root(fc1["in"][0]) == "x"
        elif folded is False:   # between the two, the norm keeps its own launch (the tiled kernel's prologue is the slower choice)
            assert [o["aten"] for o in g.ops] == ["layer_norm.default", "linear.default", "linear.default"] and "ln_in" not in fc1["attrs"]
        else:           # a wide batch: no pass for the norm at all -- statistics of the input rows, fc1 on the raw rows
            assert [o["aten"] for o in g.ops] == ["rowstats", "linear.default", "linear.default"] and "ln_in" not in fc1["attrs"]
            assert fc1["attrs"]["lnf"] == g.ops[0]["out"] and fc1["attrs"]["epilogue"] == "gelu" and g.root(fc1["in"][0]) == "x"


def test_norm_over_a_permuted_view_keeps_its_pass():
    """The folded form reads the norm's input rows as the GEMM's operand: a channels-first tensor permuted in front of the
    norm has no such rows, so the norm stays an op."""
    import torch
    import torch.nn as nn
    from juliavision_amd import graph as G

    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.ln, self.fc = nn.LayerNorm(256), nn.Linear(256, 512)

        def forward(self, x):                       # (B, C, T)
            return self.fc(self.ln(x.permute(0, 2, 1)))

    ep = torch.export.export(M().eval().half(), (torch.randn(1, 256, 300).half(),))
    g = G.optimize(G.Graph.load(G.convert(ep, "m")))
    assert [o["aten"] for o in g.ops] == ["layer_norm.default", "linear.default"] and not any("lnf" in o["attrs"] for o in g.ops)


@pytest.mark.gpu
def test_decode_sized_norm_prologue_runs_on_the_kernels(ctx):
    import torch
    from juliavision_amd import graph as G
    m = _mlp(seed=2)
    x = torch.randn(1, 4, 256).half()
    ep = torch.export.export(m, (x,))
    g = G.optimize(G.Graph.load(G.convert(ep, "mlp")))
    assert g.op("linear")["attrs"].get("ln_in") is True
    run = G.Executor(g, {k: v for k, v in m.state_dict().items()}, ctx)
    got = run(x.cuda())
    torch.cuda.synchronize()
    with torch.no_grad():
        want = m.float()(x.float())
    assert_parity(got.float().cpu().numpy(), want.numpy(), what="decode-sized norm prologue from an exported graph")


@pytest.mark.gpu
def test_executor_refuses_what_it_cannot_run(ctx):
    import torch
    from juliavision_amd import graph as G

    class M(torch.nn.Module):
        def forward(self, x):
            return torch.tanh(x)

    ep = torch.export.export(M(), (torch.randn(2, 8).half(),))
    with pytest.raises(G.UnsupportedOp, match="tanh"):
        G.Executor(G.Graph.load(G.convert(ep, "m")), {}, ctx)
    ep2, _ = _export(_block())
    g = G.fold_activations(G.Graph.load(G.convert(ep2, "block")))   # attention output still needs a copy for its reshape
    run = G.Executor(g, _block().state_dict(), ctx)
    with pytest.raises(G.UnsupportedOp, match="needs a copy"):
        run(torch.randn(1, 70, 128).half().cuda())


@pytest.mark.gpu
def test_exported_upsampler_runs_transposed_and_lifted_1d_convolutions(ctx):
    """aten::convolution with arg6 set is the transposed convolution and a one-element stride list is the 1-D
    layer lifted to a singleton second axis (runop! for convolution.default, ops.jl:1114-1200)."""
    import torch
    from juliavision_amd import graph as G

    class Up(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up = torch.nn.ConvTranspose2d(32, 16, 2, 2)            # kernel == stride: GEMM + pixel shuffle
            self.c = torch.nn.Conv2d(16, 16, 3, padding=1)
            self.u1 = torch.nn.ConvTranspose1d(16, 8, 4, 2, 1)          # overlapping: the gather
            self.c1 = torch.nn.Conv1d(8, 8, 3, padding=1)

        def forward(self, x):
            y = self.c(self.up(x))
            return self.c1(self.u1(y.flatten(2)))

    torch.manual_seed(5)
    m = Up().eval().half()
    x = torch.randn(1, 32, 8, 8).half()
    ep = torch.export.export(m, (x,)).run_decompositions()
    g = G.Graph.load(G.convert(ep, "up"))
    assert [o["aten"] for o in g.ops] == ["convolution.default"] * 4
    assert [bool(o["attrs"]["arg6"]) for o in g.ops] == [True, False, True, False]
    run = G.Executor(g, m.state_dict(), ctx)
    with torch.no_grad():
        want = m.float()(x.float()).numpy()
    got = run(x.cuda())
    torch.cuda.synchronize()
    assert tuple(got.shape) == want.shape == (1, 8, 512)
    assert_parity(got.float().cpu().numpy(), want, what="exported upsampler")


def _decomposed(m, keep_sdpa=True):
    """The block exported and lowered to core ops as the reference's exporter does (export_graphs.py:277-279):
    linear becomes addmm/mm over permuted weights, layer_norm native_layer_norm.  On a CPU the composite
    attention op would be lowered to its matmul + softmax form; keeping it stands in for the fused op an
    accelerator export holds."""
    import torch
    ep, x = _export(m)
    table = torch.export.default_decompositions()
    if keep_sdpa:
        table.pop(torch.ops.aten.scaled_dot_product_attention.default, None)
    return ep.run_decompositions(table), x


def _as_backend_attention(d, name):
    """Rewrite the dictionary's composite attention op into a tuple-returning backend form with the same
    operands, as `_scaled_dot_product_flash_attention` / `_efficient_attention` appear in accelerator exports."""
    import copy
    d = copy.deepcopy(d)
    op = next(o for o in d["ops"] if o["aten"] == "scaled_dot_product_attention.default")
    old = op["id"]
    b = next(b for b in d["buffers"] if b["id"] == old)
    op["aten"] = name
    op["attrs"] = {"arg3": 0.0, "arg4": False} if "flash" in name else {"arg4": True, "arg5": 0.0, "arg6": False}
    tup = {"id": old + "_tuple", "kind": "transient", "shapes": [b["shape"], [1, 2, 70], None], "dtypes": [b["dtype"], "float32", None],
           "live": b.get("live")}
    op["id"] = op["out"] = tup["id"]
    b.update(kind="view", of=tup["id"], op="<built-in function getitem>", attrs={"arg1": 0})
    d["buffers"].append(tup)
    return d


def test_decomposed_export_folds_like_the_composite_one():
    from juliavision_amd import graph as G
    ep, _ = _decomposed(_block())
    d = G.convert(ep, "block")
    aten = [o["aten"] for o in d["ops"]]
    assert aten.count("addmm.default") == 5 and aten.count("mm.default") == 1 and aten.count("native_layer_norm.default") == 2
    g = G.optimize(G.Graph.load(d))
    assert [o["aten"] for o in g.ops].count("gelu.default") == 0 and len(g.ops) == 6
    # neither norm is left: the first became a pass over x for its row statistics, the second rides in the out-projection's store
    assert [o["aten"] for o in g.ops].count("native_layer_norm.default") == 0 and g.ops[0]["aten"] == "rowstats"
    assert sum("stats_out" in o["attrs"] for o in g.ops) == 1 and sum("lnf" in o["attrs"] for o in g.ops) == 2
    fc1 = next(o for o in g.ops if o["attrs"].get("epilogue") == "gelu")
    assert fc1["aten"] == "addmm.default" and g.root("gelu") == fc1["id"]       # gelu read the addmm through a view
    assert sum("residual" in o["attrs"] for o in g.ops) == 2
    for name in ("_scaled_dot_product_flash_attention.default", "_scaled_dot_product_efficient_attention.default"):
        g2 = G.optimize(G.Graph.load(_as_backend_attention(d, name)))
        att = next(o for o in g2.ops if o["aten"] == name)
        assert att["attrs"]["token_major"] is True and len(g2.ops) == 6


@pytest.mark.gpu
@pytest.mark.parametrize("attention", ["scaled_dot_product_attention.default", "_scaled_dot_product_flash_attention.default",
                                       "_scaled_dot_product_efficient_attention.default"])
def test_decomposed_export_runs_on_the_kernels(ctx, attention):
    import torch
    from juliavision_amd import graph as G
    m = _block(seed=4)
    ep, x = _decomposed(m)
    d = G.convert(ep, "block")
    if attention != "scaled_dot_product_attention.default":
        d = _as_backend_attention(d, attention)
    run = G.Executor(G.optimize(G.Graph.load(d)), m.state_dict(), ctx)
    with torch.no_grad():
        want = m.float()(x.float()).numpy()
    got = run(x.cuda())
    torch.cuda.synchronize()
    assert_parity(got.float().cpu().numpy(), want, what=f"decomposed block, {attention}")


@pytest.mark.gpu
def test_executor_takes_weights_from_a_safetensors_file(ctx, tmp_path):
    """Graph JSON + weights file, the two artifacts the reference's Model(dir, weights) is built from (driver.jl:165-168)."""
    import torch
    from safetensors.torch import save_file
    from juliavision_amd import graph as G
    from juliavision_amd import safetensors as ST
    m = _block(seed=6)
    ep, x = _export(m)
    (tmp_path / "block.json").write_text(json.dumps(G.convert(ep, "block")))
    save_file({k: v.float().contiguous() for k, v in m.state_dict().items()}, str(tmp_path / "block.safetensors"))   # stored in fp32
    g = G.optimize(G.Graph.load(json.loads((tmp_path / "block.json").read_text())))
    run = G.Executor(g, ST.load_to(str(tmp_path / "block.safetensors"), "cuda", torch.float16), ctx)
    with torch.no_grad():
        want = m.float()(x.float()).numpy()
    assert_parity(run(x.cuda()).float().cpu().numpy(), want, what="block from graph JSON + safetensors")


def _written_out_attention(style, d=128, heads=2, seed=0, return_probs=False):
    """Attention as the models that never reach ``scaled_dot_product_attention`` write it: DINOv2's (q scaled
    first, ``@``, softmax, ``@``; Depth Anything's backbone) or the eager Hugging Face form (scores divided by
    sqrt(E) after the product)."""
    import torch
    import torch.nn as nn

    class Attn(nn.Module):
        def __init__(self):
            super().__init__()
            self.h, self.scale = heads, (d // heads) ** -0.5
            self.qkv, self.proj = nn.Linear(d, 3 * d), nn.Linear(d, d)

        def forward(self, x):
            B, N, C = x.shape
            qkv = self.qkv(x).reshape(B, N, 3, self.h, C // self.h).permute(2, 0, 3, 1, 4)
            if style == "dinov2":
                q, k, v = qkv[0] * self.scale, qkv[1], qkv[2]
                attn = (q @ k.transpose(-2, -1)).softmax(dim=-1)
                y = (attn @ v).transpose(1, 2).reshape(B, N, C)
            else:
                attn = torch.matmul(qkv[0], qkv[1].transpose(-1, -2)) / (C // self.h) ** 0.5
                attn = torch.nn.functional.softmax(attn, dim=-1)
                y = torch.matmul(attn, qkv[2]).permute(0, 2, 1, 3).contiguous().view(B, N, C)
            return (self.proj(y), attn) if return_probs else self.proj(y)

    torch.manual_seed(seed)
    return Attn().eval().half()


@pytest.mark.parametrize("style", ["dinov2", "hf_eager"])
@pytest.mark.parametrize("B", [1, 2])
def test_written_out_attention_folds_into_the_fused_op(style, B):
    """24 bmm + 12 _softmax is how the reference's Depth Anything graph holds its attention
    (DepthAnythingRunner.jl:38-42); with a batch the export also copies the operands contiguous first."""
    import torch
    from juliavision_amd import graph as G
    m = _written_out_attention(style)
    ep = torch.export.export(m, (torch.randn(B, 70, 128).half(),)).run_decompositions()
    d = G.convert(ep, "attn")
    aten = [o["aten"] for o in d["ops"]]
    assert aten.count("bmm.default") == 2 and aten.count("_softmax.default") == 1
    g = G.optimize(G.Graph.load(d))
    assert [o["aten"] for o in g.ops] == ["addmm.default", "scaled_dot_product_attention.default", "addmm.default"], g.notes
    att = g.ops[1]
    assert att["attrs"]["scale"] == pytest.approx(0.125) and att["attrs"]["token_major"] is True
    assert [g.buffers[i]["shape"] for i in att["in"]] == [[B, 2, 70, 64]] * 3


def test_attention_whose_probabilities_are_returned_stays_as_it_is():
    import torch
    from juliavision_amd import graph as G
    m = _written_out_attention("hf_eager", return_probs=True)
    ep = torch.export.export(m, (torch.randn(1, 70, 128).half(),)).run_decompositions()
    g = G.optimize(G.Graph.load(G.convert(ep, "attn")))
    assert [o["aten"] for o in g.ops].count("bmm.default") == 2 and not any("sdpa" in n for n in g.notes)


@pytest.mark.gpu
@pytest.mark.parametrize("style,B", [("dinov2", 1), ("dinov2", 2), ("hf_eager", 1)])
def test_written_out_attention_runs_on_the_fused_kernel(ctx, style, B):
    import torch
    from juliavision_amd import graph as G
    m = _written_out_attention(style, seed=3)
    x = torch.randn(B, 70, 128).half()
    ep = torch.export.export(m, (x,)).run_decompositions()
    run = G.Executor(G.optimize(G.Graph.load(G.convert(ep, "attn"))), m.state_dict(), ctx)
    with torch.no_grad():
        want = m.float()(x.float()).numpy()
    got = run(x.cuda())
    torch.cuda.synchronize()
    assert_parity(got.float().cpu().numpy(), want, what=f"written-out attention, {style}, batch {B}")


@pytest.mark.gpu
def test_bmm_runs_on_the_batched_gemm(ctx):
    """aten::bmm on its own (ops.jl:1393-1399 -> batchedmatmul!)."""
    import torch
    from juliavision_amd import graph as G

    class M(torch.nn.Module):
        def forward(self, a, b):
            return torch.bmm(a, b)

    a, b = torch.randn(6, 70, 64).half(), torch.randn(6, 64, 40).half()
    ep = torch.export.export(M(), (a, b)).run_decompositions()
    run = G.Executor(G.Graph.load(G.convert(ep, "bmm")), {}, ctx)
    got = run(a.cuda(), b.cuda())
    torch.cuda.synchronize()
    assert_parity(got.float().cpu().numpy(), torch.bmm(a.float(), b.float()).numpy(), what="bmm")


def _dinov2_like(d=128, heads=2, layers=2, patch=14, image=70, seed=0):
    """A ViT written the way DINOv2 (the backbone of the reference's Depth Anything model, config 3) is: patch
    embedding by a strided convolution, class token concatenated in front, learned position embedding, pre-LN blocks
    with written-out attention and LayerScale on both branches, a final norm."""
    import torch
    import torch.nn as nn

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.h, self.scale = heads, (d // heads) ** -0.5
            self.norm1, self.norm2 = nn.LayerNorm(d, eps=1e-6), nn.LayerNorm(d, eps=1e-6)
            self.qkv, self.proj = nn.Linear(d, 3 * d), nn.Linear(d, d)
            self.fc1, self.fc2 = nn.Linear(d, 4 * d), nn.Linear(4 * d, d)
            self.ls1, self.ls2 = nn.Parameter(torch.rand(d) + 0.5), nn.Parameter(torch.rand(d) + 0.5)

        def attn(self, x):
            B, N, C = x.shape
            qkv = self.qkv(x).reshape(B, N, 3, self.h, C // self.h).permute(2, 0, 3, 1, 4)
            q, k, v = qkv[0] * self.scale, qkv[1], qkv[2]
            a = (q @ k.transpose(-2, -1)).softmax(dim=-1)
            return self.proj((a @ v).transpose(1, 2).reshape(B, N, C))

        def forward(self, x):
            x = x + self.attn(self.norm1(x)) * self.ls1
            return x + self.fc2(torch.nn.functional.gelu(self.fc1(self.norm2(x)))) * self.ls2

    class ViT(nn.Module):
        def __init__(self):
            super().__init__()
            n = (image // patch) ** 2
            self.patch_embed = nn.Conv2d(3, d, patch, patch)
            self.cls_token, self.pos_embed = nn.Parameter(torch.randn(1, 1, d) * 0.1), nn.Parameter(torch.randn(1, n + 1, d) * 0.1)
            self.blocks = nn.ModuleList([Block() for _ in range(layers)])
            self.norm = nn.LayerNorm(d, eps=1e-6)

        def forward(self, img):
            x = self.patch_embed(img).flatten(2).transpose(1, 2)
            x = torch.cat((self.cls_token.expand(x.shape[0], -1, -1), x), dim=1) + self.pos_embed
            for b in self.blocks:
                x = b(x)
            return self.norm(x)

    torch.manual_seed(seed)
    return ViT().eval().half()


def test_dinov2_like_encoder_folds_to_five_calls_per_block():
    import torch
    from juliavision_amd import graph as G
    m = _dinov2_like()
    ep = torch.export.export(m, (torch.randn(1, 3, 70, 70).half(),)).run_decompositions()
    d = G.convert(ep, "vit")
    aten = [o["aten"] for o in d["ops"]]
    assert aten.count("bmm.default") == 4 and aten.count("_softmax.default") == 2 and aten.count("cat.default") == 1
    g = G.optimize(G.Graph.load(d))
    left = [o["aten"] for o in g.ops]
    # the patch embedding (convolution written as tokens, class row, position embedding: one op), first norm; per
    # block: qkv, attention, projection, fc1, fc2 -- the other norms ride in the GEMM that writes their input,
    # LayerScale in the weights, residuals in the stores
    assert left == ["patch_tokens", "native_layer_norm.default"] + \
        ["addmm.default", "scaled_dot_product_attention.default", "addmm.default", "addmm.default", "addmm.default"] * 2, (left, g.notes)
    assert sum("colscale" in o["attrs"] for o in g.ops) == 4 and sum("residual" in o["attrs"] for o in g.ops) == 4
    assert sum("ln_out" in o["attrs"] for o in g.ops) == 4


def test_division_by_a_weight_vector_is_not_folded_as_layerscale():
    """Only ``linear(x) * g`` is a column scale of the weights; ``linear(x) / g`` and ``g / linear(x)`` are not, and
    stay in the graph as written (there the executor refuses them by name instead of computing ``W * g``)."""
    import torch
    import torch.nn as nn
    from juliavision_amd import graph as G

    class M(nn.Module):
        def __init__(self, mode):
            super().__init__()
            self.lin, self.g, self.mode = nn.Linear(16, 24), nn.Parameter(torch.rand(24) + 0.5), mode

        def forward(self, x):
            y = self.lin(x)
            return y * self.g if self.mode == "mul" else y / self.g if self.mode == "div" else self.g / y

    for mode in ("mul", "div", "rdiv"):
        ep = torch.export.export(M(mode).eval().half(), (torch.randn(5, 16).half(),)).run_decompositions()
        g = G.optimize(G.Graph.load(G.convert(ep, mode)))
        folded = [o for o in g.ops if "colscale" in o["attrs"]]
        left = [o["aten"] for o in g.ops]
        if mode == "mul":
            assert len(folded) == 1 and "mul.Tensor" not in left, (left, g.notes)
        else:
            assert not folded and "div.Tensor" in left, (mode, left, g.notes)


def test_patch_embedding_whose_feature_map_is_also_a_result_is_not_folded():
    """The fold drops the channel-major convolution result; a graph that returns it keeps the three ops."""
    import torch
    import torch.nn as nn
    from juliavision_amd import graph as G

    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.pe, self.cls, self.pos = nn.Conv2d(3, 32, 8, 8), nn.Parameter(torch.zeros(1, 1, 32)), nn.Parameter(torch.zeros(1, 10, 32))

        def forward(self, img):
            f = self.pe(img)
            x = f.flatten(2).transpose(1, 2)
            return torch.cat((self.cls.expand(x.shape[0], -1, -1), x), dim=1) + self.pos, f

    ep = torch.export.export(M().eval().half(), (torch.randn(1, 3, 24, 24).half(),)).run_decompositions()
    g = G.optimize(G.Graph.load(G.convert(ep, "pe")))
    assert [o["aten"] for o in g.ops] == ["convolution.default", "cat.default", "add.Tensor"], g.notes


@pytest.mark.gpu
@pytest.mark.parametrize("B,image", [(1, 70), (2, 70), (1, 126), (2, 126)])
def test_dinov2_like_encoder_runs_on_the_kernels(ctx, B, image):
    """26 token rows per image at 70 x 70 (the norms keep a pass or ride as a GEMM's second result), 82 at 126 x 126 (the
    norms between GEMMs are folded away: LayerScale, residual and row statistics in one store, the next GEMM on the raw rows)."""
    import torch
    from juliavision_amd import graph as G
    m = _dinov2_like(seed=5, image=image)
    x = torch.rand(B, 3, image, image).half()
    ep = torch.export.export(m, (x,)).run_decompositions()
    g = G.optimize(G.Graph.load(G.convert(ep, "vit")))
    assert g.ops[0]["aten"] == "patch_tokens"
    tokens = (image // 14) ** 2 + 1
    assert any("lnf" in o["attrs"] for o in g.ops) == (B * tokens >= 64)
    run = G.Executor(g, m.state_dict(), ctx)
    with torch.no_grad():
        want = m.float()(x.float()).numpy()
    got = run(x.cuda())
    torch.cuda.synchronize()
    assert got.shape == (B, tokens, 128)
    assert_parity(got.float().cpu().numpy(), want, what="DINOv2-like encoder from its exported graph")


@pytest.mark.gpu
@pytest.mark.parametrize("style,B", [("dinov2", 1), ("dinov2", 2), ("hf_eager", 2)])
def test_written_out_attention_runs_as_written_too(ctx, style, B):
    """Without the rewrite the same graph runs op by op -- two batched GEMMs around the row softmax, the reference's
    two-GEMM attention (sdpa_coopmat!, attention.jl:675-705) -- and lands where the fused kernel does."""
    import torch
    from juliavision_amd import graph as G
    m = _written_out_attention(style, seed=7)
    x = torch.randn(B, 70, 128).half()
    ep = torch.export.export(m, (x,)).run_decompositions()
    d = G.convert(ep, "attn")
    plain = G.Executor(G.Graph.load(d), m.state_dict(), ctx)
    assert [o["aten"] for o in plain.g.ops].count("bmm.default") == 2
    fused = G.Executor(G.optimize(G.Graph.load(d)), m.state_dict(), ctx)
    with torch.no_grad():
        want = m.float()(x.float()).numpy()
    got_plain, got_fused = plain(x.cuda()).float().cpu().numpy(), fused(x.cuda()).float().cpu().numpy()
    assert_parity(got_plain, want, what=f"{style} as written")
    assert_parity(got_plain, got_fused, what=f"{style} as written vs fused")


@pytest.mark.gpu
def test_attention_that_returns_its_probabilities_runs(ctx):
    import torch
    from juliavision_amd import graph as G
    m = _written_out_attention("hf_eager", seed=8, return_probs=True)
    x = torch.randn(1, 70, 128).half()
    ep = torch.export.export(m, (x,)).run_decompositions()
    run = G.Executor(G.optimize(G.Graph.load(G.convert(ep, "attn"))), m.state_dict(), ctx)
    with torch.no_grad():
        want_y, want_p = (t.numpy() for t in m.float()(x.float()))
    y, p = run(x.cuda())
    assert_parity(y.float().cpu().numpy(), want_y, what="output")
    assert_parity(p.float().cpu().numpy(), want_p, what="probabilities")


def _whisper_like_encoder(d=128, heads=2, layers=2, mels=16, frames=60, seed=0):
    """An audio encoder written the way Whisper's is (the model of configs 1, 2 and 5): two 1-D convolutions with GELU
    (the second of stride 2), learned positions, pre-LN layers whose query projection is multiplied by
    head_dim ** -0.5 ahead of a fused attention with scale 1, k_proj without bias, the fp16 clamp after each layer,
    a final norm."""
    import torch
    import torch.nn as nn
    import torch.nn.functional as F

    class Layer(nn.Module):
        def __init__(self):
            super().__init__()
            self.h, self.scaling = heads, (d // heads) ** -0.5
            self.ln1, self.ln2 = nn.LayerNorm(d), nn.LayerNorm(d)
            self.q, self.k, self.v, self.o = nn.Linear(d, d), nn.Linear(d, d, bias=False), nn.Linear(d, d), nn.Linear(d, d)
            self.fc1, self.fc2 = nn.Linear(d, 4 * d), nn.Linear(4 * d, d)

        def forward(self, x):
            B, T, D = x.shape
            y = self.ln1(x)
            sp = lambda t: t.view(B, T, self.h, D // self.h).transpose(1, 2)
            a = F.scaled_dot_product_attention(sp(self.q(y) * self.scaling), sp(self.k(y)), sp(self.v(y)), scale=1.0)
            x = x + self.o(a.transpose(1, 2).reshape(B, T, D))
            x = x + self.fc2(F.gelu(self.fc1(self.ln2(x))))
            return torch.clamp(x, min=-64504.0, max=64504.0)

    class Encoder(nn.Module):
        def __init__(self):
            super().__init__()
            self.conv1, self.conv2 = nn.Conv1d(mels, d, 3, padding=1), nn.Conv1d(d, d, 3, stride=2, padding=1)
            self.pos = nn.Parameter(torch.randn(frames // 2, d) * 0.1)
            self.layers = nn.ModuleList([Layer() for _ in range(layers)])
            self.ln_post = nn.LayerNorm(d)

        def forward(self, mel):
            x = F.gelu(self.conv2(F.gelu(self.conv1(mel))))
            x = x.permute(0, 2, 1) + self.pos
            for l in self.layers:
                x = l(x)
            return self.ln_post(x)

    torch.manual_seed(seed)
    return Encoder().eval().half()


def _export_keeping_sdpa(m, x):
    import torch
    table = torch.export.default_decompositions()
    table.pop(torch.ops.aten.scaled_dot_product_attention.default, None)
    return torch.export.export(m, (x,)).run_decompositions(table)


def test_whisper_like_encoder_rewrites():
    import torch
    from juliavision_amd import graph as G
    m = _whisper_like_encoder()
    d = G.convert(_export_keeping_sdpa(m, torch.randn(1, 16, 60).half()), "enc")
    aten = [o["aten"] for o in d["ops"]]
    assert aten.count("clamp.default") == 2 and aten.count("mul.Tensor") == 2 and aten.count("gelu.default") == 4
    g = G.optimize(G.Graph.load(d))
    left = [o["aten"] for o in g.ops]
    # stem: conv, gelu, conv, gelu, + positions, first norm; per layer q/k/v (one launch), attention, out-projection, fc1, fc2
    assert left.count("mul.Tensor") == 0 and left.count("gelu.default") == 2, (left, g.notes)
    # the clamp rides in the second MLP GEMM's store, and with it the norm that reads the clamped stream
    assert left.count("clamp.default") == 0 and left.count("native_layer_norm.default") == 1
    fc2 = [o for o in g.ops if o["attrs"].get("clamp") is not None]
    assert len(fc2) == 2 and all(o["attrs"]["clamp"] == 64504.0 and "residual" in o["attrs"] and "ln_out" in o["attrs"] for o in fc2)
    grp = [o for o in g.ops if o["aten"] == "linear_group"]
    assert len(grp) == 2 and all(len(o["attrs"]["members"]) == 3 for o in grp)                  # q, k, v of each layer: one launch
    assert [m["colscale"] for m in grp[0]["attrs"]["members"]] == [pytest.approx(0.125), None, None]   # the constant after q_proj
    assert sum(o["attrs"].get("epilogue") == "gelu" for o in g.ops) == 2 and sum("residual" in o["attrs"] for o in g.ops) == 4


def test_whisper_like_encoder_with_enough_rows_loses_its_norms():
    """160 frames -> 80 token rows: every norm but the last (the graph's result) is folded away.  The first layer's reads the
    stem's output (an add of the positions: no GEMM wrote it) and gets a rowstats op; every other one takes the statistics
    the GEMM before it leaves next to its residual add and clamp."""
    import torch
    from juliavision_amd import graph as G
    m = _whisper_like_encoder(frames=160)
    g = G.optimize(G.Graph.load(G.convert(_export_keeping_sdpa(m, torch.randn(1, 16, 160).half()), "enc")))
    left = [o["aten"] for o in g.ops]
    assert left.count("rowstats") == 1 and left.count("native_layer_norm.default") == 0 and left.count("clamp.default") == 0, (left, g.notes)
    grp = [o for o in g.ops if o["aten"] == "linear_group"]
    assert len(grp) == 2 and all(o["attrs"].get("lnf") and len(o["attrs"]["members"]) == 3 for o in grp)
    assert grp[0]["attrs"]["lnf"] == g.ops[left.index("rowstats")]["out"]
    writers = [o for o in g.ops if "stats_out" in o["attrs"]]
    assert len(writers) == 3 and all("residual" in o["attrs"] for o in writers)              # proj, fc2 of layer 0; proj of layer 1
    assert writers[1]["attrs"]["clamp"] == 64504.0 and grp[1]["attrs"]["lnf"] == writers[1]["attrs"]["stats_out"]
    fc1 = [o for o in g.ops if o["attrs"].get("epilogue") == "gelu" and o["aten"] != "convolution.default"]
    assert [o["attrs"].get("lnf") for o in fc1] == [writers[0]["attrs"]["stats_out"], writers[2]["attrs"]["stats_out"]]
    last = g.ops[-1]                                                                           # the final norm is returned: it stays a result
    assert last["attrs"].get("ln_out") is not None and last["attrs"]["clamp"] == 64504.0 and "stats_out" not in last["attrs"]


@pytest.mark.gpu
@pytest.mark.parametrize("frames", [60, 160])
def test_whisper_like_encoder_runs_on_the_kernels(ctx, frames):
    import torch
    from juliavision_amd import graph as G
    m = _whisper_like_encoder(seed=9, frames=frames)
    x = torch.randn(1, 16, frames).half()
    run = G.Executor(G.optimize(G.Graph.load(G.convert(_export_keeping_sdpa(m, x), "enc"))), m.state_dict(), ctx)
    with torch.no_grad():
        want = m.float()(x.float()).numpy()
    got = run(x.cuda())
    torch.cuda.synchronize()
    assert got.shape == (1, frames // 2, 128)
    assert_parity(got.float().cpu().numpy(), want, what="Whisper-like encoder from its exported graph")


@pytest.mark.gpu
def test_executor_replays_as_one_captured_graph(ctx):
    """Executor.replayable: the whole op list captured once; replays follow the input tensor's contents and match the
    eager run every time (several replays with eager work and synchronisations between them)."""
    import torch
    from juliavision_amd import graph as G
    m = _dinov2_like(seed=11)
    x = torch.rand(1, 3, 70, 70).half().cuda()
    ep = torch.export.export(m, (x.cpu(),)).run_decompositions()
    run = G.Executor(G.optimize(G.Graph.load(G.convert(ep, "vit"))), m.state_dict(), ctx)
    replay, out = run.replayable(x)
    for seed in (1, 2, 3):
        torch.manual_seed(seed)
        x.copy_(torch.rand(1, 3, 70, 70).half())
        replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = run(x).clone()                       # eager, same tensors
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {seed} differs from the eager run"
        with torch.no_grad():
            ref = m.float()(x.float().cpu()).numpy()
        assert_parity(got.float().cpu().numpy(), ref, what=f"replay {seed}")


def _conv_relu_stack(seed=0):
    import torch
    import torch.nn as nn

    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.c1, self.c2, self.c3 = nn.Conv2d(16, 32, 3, padding=1), nn.Conv2d(32, 32, 1), nn.ConvTranspose2d(32, 8, 2, stride=2)

        def forward(self, x):
            y = torch.relu(self.c1(x))                      # folds: the convolution's own act
            y = torch.nn.functional.gelu(self.c2(y))        # gelu after a convolution has no such slot: stays an op
            return torch.relu(self.c3(y))                   # nor has the transposed convolution

    torch.manual_seed(seed)
    return M().eval().half()


def test_relu_after_a_convolution_becomes_its_act():
    import torch
    from juliavision_amd import graph as G
    m = _conv_relu_stack()
    g = G.optimize(G.Graph.load(G.convert(torch.export.export(m, (torch.randn(1, 16, 24, 24).half(),)).run_decompositions(), "convs")))
    left = [o["aten"] for o in g.ops]
    assert left.count("relu.default") == 1 and left.count("gelu.default") == 1 and left.count("convolution.default") == 3, (left, g.notes)
    convs = [o for o in g.ops if o["aten"] == "convolution.default"]
    assert [o["attrs"].get("epilogue") for o in convs] == ["relu", None, None]


@pytest.mark.gpu
def test_convolution_with_folded_relu_runs_on_the_kernels(ctx):
    import torch
    from juliavision_amd import graph as G
    m = _conv_relu_stack(seed=3)
    x = torch.randn(1, 16, 24, 24).half()
    run = G.Executor(G.optimize(G.Graph.load(G.convert(torch.export.export(m, (x,)).run_decompositions(), "convs"))), m.state_dict(), ctx)
    with torch.no_grad():
        want = m.float()(x.float()).numpy()
    got = run(x.cuda())
    torch.cuda.synchronize()
    assert_parity(got.float().cpu().numpy(), want, what="conv + relu folded, conv + gelu, transposed conv + relu")


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["composite", "decomposed"])
def test_exported_block_matches_the_oracle_composition(ctx, mode):
    """The exported block against the composition of the oracle's CPU kernels that the hand-composed encoder layer is held
    to (layer norm, one rounding per GEMM, activation on the rounded value, residual with one more rounding, three-pass
    attention), fed the module's own weights: the graph route and the oracle agree, not only the graph route and torch."""
    import numpy as np
    import torch
    import oracle
    from juliavision_amd import graph as G
    from test_configs_gpu import _oracle_layer
    d, heads, ffn, T = 128, 2, 256, 70
    m = _block(d, heads, ffn, seed=5)
    with torch.no_grad():
        m.k.bias = torch.nn.Parameter(torch.zeros(d).half())          # the oracle's packed q/k/v bias needs all three
    ep, x = _export(m, T, d) if mode == "composite" else _decomposed(m)
    run = G.Executor(G.optimize(G.Graph.load(G.convert(ep, "block"))), m.state_dict(), ctx)
    got = run(x.cuda())
    torch.cuda.synchronize()
    np16 = lambda t: t.detach().cpu().numpy().astype(np.float16)
    kf = lambda lin: np.ascontiguousarray(np16(lin.weight).T)           # torch [F][K] -> the oracle's [K][F]
    h = {"wqkv": np.concatenate([kf(m.q), kf(m.k), kf(m.v)], axis=1), "bqkv": np.concatenate([np16(m.q.bias), np16(m.k.bias), np16(m.v.bias)]),
         "wo": kf(m.o), "bo": np16(m.o.bias), "w1": kf(m.fc1), "b1": np16(m.fc1.bias), "w2": kf(m.fc2), "b2": np16(m.fc2.bias),
         "ln1_g": np16(m.ln1.weight), "ln1_b": np16(m.ln1.bias), "ln2_g": np16(m.ln2.weight), "ln2_b": np16(m.ln2.bias)}
    x16 = np16(x)[0]
    want = _oracle_layer(h, x16, heads, 1e-5)
    assert_parity(got.float().cpu().numpy()[0], want, what=f"exported block ({mode}) against the oracle's composition")
    assert_parity(got.float().cpu().numpy()[0] - x16.astype(np.float32), want.astype(np.float32) - x16.astype(np.float32),
                  what="the block's update alone")
