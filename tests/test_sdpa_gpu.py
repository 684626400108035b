"""Attention parity on the GPU through the C ABI.

Oracles: the three-pass KA-CPU form (attention.jl:46-112) and the composed
Float32 softmax(QK^T)V (test_flash.jl:13-24) for the fused kernel, which the
reference marks cpu=false.  Gate: max rel <= 1e-2, cosine >= 0.9999; the
reference's own fp16 tolerance is 5e-3 of max (test_flash.jl:142)."""
import numpy as np
import pytest

import oracle
from util import assert_parity, poison, to_dev, to_host

pytestmark = pytest.mark.gpu


def _qkv(B, H, Lq, Lk, E, seed, std=1.0):
    q = oracle.randn_f16((B, H, Lq, E), seed, 0, std)
    k = oracle.randn_f16((B, H, Lk, E), seed + 1, 0, std)
    v = oracle.randn_f16((B, H, Lk, E), seed + 2, 0, std)
    return q, k, v


def _check(ctx, q, k, v, *, bias=None, scale=None, kv_len=None, out_dtype="f16", expect=None, what=""):
    import torch
    import juliavision_amd as jv
    dq, dk, dv = (a if isinstance(a, torch.Tensor) else to_dev(a) for a in (q, k, v))
    hq, hk, hv = (to_host(a) if isinstance(a, torch.Tensor) else a for a in (q, k, v))
    db = None if bias is None else to_dev(bias)
    dl = None if kv_len is None else torch.tensor(kv_len, dtype=torch.int32, device="cuda")
    plan = jv.sdpaplan(ctx, dq, dk, dv, db, scale, dl)
    if expect is not None:
        assert type(plan).__name__ == expect, f"{what}: plan {plan}"
    B, H, Lq, E = hq.shape
    out = poison(torch.empty((B, H, Lq, E), dtype=torch.float16 if out_dtype == "f16" else torch.float32, device="cuda"))
    ctx.ws.reset()
    jv.sdpa(ctx, dq, dk, dv, db, scale, out=out, kv_len=dl)
    torch.cuda.synchronize()
    got = to_host(out)
    ref32 = oracle.sdpa_ref_f32(hq, hk, hv, bias, scale, kv_len=kv_len)
    assert_parity(got, ref32, what=what + " vs composed f32")
    tp = oracle.sdpa_threepass_f16(hq, hk, hv, bias, scale, kv_len=kv_len, out_f32=(out_dtype != "f16"))
    assert_parity(got, tp, what=what + " vs three-pass")
    return got


@pytest.mark.parametrize("B,H,Lq,Lk,E", [
    (1, 2, 128, 128, 64), (1, 2, 256, 256, 64), (2, 3, 200, 137, 64), (1, 1, 64, 17, 64),
    (1, 2, 130, 23, 32), (1, 2, 128, 128, 72), (1, 1, 128, 64, 16), (1, 2, 192, 320, 128), (1, 1, 1500, 1500, 64),
])
def test_flash_shapes(ctx, B, H, Lq, Lk, E):
    q, k, v = _qkv(B, H, Lq, Lk, E, 31)
    _check(ctx, q, k, v, expect="FlashPlan", what=f"flash {B},{H},{Lq},{Lk},{E}")


@pytest.mark.parametrize("B,H,Lq,Lk,E,kw", [
    (1, 2, 256, 256, 72, {}),                              # SAM 2's windowed attention: 256 tokens, head size 72 (tools/attn_lab.jl:8-14)
    (1, 1, 300, 1000, 72, {}),                             # ragged queries and keys, a masked last block
    (2, 2, 128, 200, 80, {"kv_len": [200, 77]}),           # per-batch valid keys
    (1, 2, 130, 129, 88, {"out_dtype": "f32"}),            # one key in the last block; fp32 rows out
    (1, 1, 192, 320, 96, {}),                              # the variant's full width
    (1, 1, 128, 2048, 72, {}),                             # one query block over 32 key blocks: the keys are split over workgroups
    (1, 8, 520, 1030, 72, {}),                             # 1024 keys or more, keys not split over workgroups: eight waves on the two
    (3, 4, 300, 1153, 96, {"kv_len": [1153, 0, 1025], "out_dtype": "f32"}),   # halves of a 128-key stage, 96 wide; ragged last stage,
    (1, 16, 2048, 1100, 80, {}),                           # per-batch lengths; a grid over more than half of the chip
])
def test_flash_head_sizes_65_to_96(ctx, B, H, Lq, Lk, E, kw):
    """Head sizes in (64, 96] run the 96-wide instance of the fused kernel (six k-steps in the first product, three
    32-wide output tiles), not the 128-wide one."""
    q, k, v = _qkv(B, H, Lq, Lk, E, 61)
    _check(ctx, q, k, v, expect="FlashPlan", what=f"flash {B},{H},{Lq},{Lk},{E}", **kw)


def test_wide_heads_key_halves_follow_growing_scores(ctx):
    """The 96-wide key-halves form moves its reference point like the others: keys far above everything before them, in
    the first and in the second half of a stage."""
    q, k, v = _qkv(1, 8, 300, 1200, 72, 303)
    q = (q.astype(np.float32) * 3.0).astype(np.float16)
    k = k.copy()
    k[:, :, 70:75] *= np.float16(4.0)
    k[:, :, 150:152] *= np.float16(8.0)
    k[:, :, 1100] *= np.float16(10.0)
    got = _check(ctx, q, k, v, expect="FlashPlan", what="growing scores, 96-wide key halves")
    assert np.all(np.isfinite(got))


def test_flash_small_inputs_and_f32_out(ctx):
    # the reference's own test inputs: randn * 0.2 (test_flash.jl:41-43)
    q, k, v = _qkv(2, 2, 128, 128, 72, 41, std=0.2)
    _check(ctx, q, k, v, out_dtype="f32", expect="FlashPlan", what="flash 0.2 f32")


def test_reference_closed_form_inputs(ctx):
    # 0.4*sin / cos / sin over ranges 9, 7, 5 (test_coopmat_attention.jl:54-55), (E,L,H,B) = (64,256,2,1)
    E, L, H, B = 64, 256, 2, 1
    n = E * L * H * B
    q = (0.4 * np.sin(np.linspace(0, 9, n))).astype(np.float16).reshape(B, H, L, E)
    k = (0.4 * np.cos(np.linspace(0, 7, n))).astype(np.float16).reshape(B, H, L, E)
    v = (0.4 * np.sin(np.linspace(0, 5, n))).astype(np.float16).reshape(B, H, L, E)
    _check(ctx, q, k, v, expect="FlashPlan", what="closed-form inputs")


def test_strided_heads_from_packed_qkv(ctx):
    """q/k/v as strided views of one packed [T][3][H][E] projection -- how the graph hands them over."""
    import torch
    T, H, E = 300, 4, 64
    packed = to_dev(oracle.randn_f16((1, T, 3, H, E), 51))
    q = packed[:, :, 0].permute(0, 2, 1, 3)
    k = packed[:, :, 1].permute(0, 2, 1, 3)
    v = packed[:, :, 2].permute(0, 2, 1, 3)
    assert not q.is_contiguous()
    _check(ctx, q, k, v, expect="FlashPlan", what="strided qkv")


def test_rows_path_small_lq_and_ragged(ctx):
    # ragged shapes of test_flash.jl:189-190 as (E,Lq,Lk,H,B): (32,23,23,8,1), (16,23,17,4,1)
    for (E, Lq, Lk, H, B) in [(32, 23, 23, 8, 1), (16, 23, 17, 4, 1), (64, 1, 448, 20, 4), (72, 5, 100, 2, 1), (20, 3, 50, 2, 2)]:
        q, k, v = _qkv(B, H, Lq, Lk, E, 61)
        _check(ctx, q, k, v, expect="RowsSDPAPlan", what=f"rows {E},{Lq},{Lk},{H},{B}")


def test_the_references_decoder_shapes_with_a_23_in_them(ctx):
    """The other two ragged shapes of test_flash.jl:189-190, SAM 2.1's mask decoder attending the image and back:
    (16,23,4096,8,1) -- 23 queries over 4096 keys, the reference's flash-decoding case (flash.jl:1288-1303), here the
    fused kernel with the keys cut over workgroups and a merge -- and (16,4096,23,8,1), 4096 queries over 23 keys
    (fewer keys than one block: a loop that counted whole blocks would run zero times)."""
    import juliavision_amd as jv
    q, k, v = _qkv(1, 8, 23, 4096, 16, 62)
    plan = jv.sdpaplan(ctx, *(to_dev(t) for t in (q, k, v)))
    assert type(plan).__name__ == "FlashPlan" and plan.nsplit > 1, plan
    _check(ctx, q, k, v, expect="FlashPlan", what="23 queries over 4096 keys")
    q, k, v = _qkv(1, 8, 4096, 23, 16, 63)
    _check(ctx, q, k, v, expect="FlashPlan", what="4096 queries over 23 keys")
    # the same few-query route with wider heads, a per-batch key count, and a key range that leaves a ragged last split
    for (E, Lq, Lk, H, B, kv) in [(64, 23, 4096, 8, 1, None), (72, 40, 1111, 4, 2, [700, 1111]), (128, 8, 600, 2, 1, None), (64, 63, 2000, 20, 1, [1999])]:
        q, k, v = _qkv(B, H, Lq, Lk, E, 64)
        _check(ctx, q, k, v, kv_len=kv, expect="FlashPlan", what=f"few queries {E},{Lq},{Lk},{H},{B}")
    # without the workspace for its partials the same call still runs (unsplit)
    q, k, v = _qkv(1, 8, 23, 4096, 16, 65)
    dq, dk, dv = (to_dev(t) for t in (q, k, v))
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    out = poison(torch.empty((1, 8, 23, 16), dtype=torch.float16, device="cuda"))
    st = lambda t: L.strides4(1, t.stride(2), t.stride(1), t.stride(0))
    rc = lib.mi_sdpa_f16(out.data_ptr(), L.F16, None, dq.data_ptr(), st(dq), dk.data_ptr(), st(dk), dv.data_ptr(), st(dv),
                         None, 0, None, None, 16, 23, 4096, 8, 1, 0.25, None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == L.OK
    torch.cuda.synchronize()
    assert_parity(to_host(out), oracle.sdpa_ref_f32(q, k, v), what="few queries, no workspace")


def test_additive_mask_and_kv_len_agree(ctx):
    """The decoder's additive 0 / finfo.min mask (B,H,1,Lk) and kv_len give the same result."""
    B, H, Lk, E = 4, 20, 448, 64
    q, k, v = _qkv(B, H, 1, Lk, E, 71)
    for pos in (3, 447):
        mask = np.where(np.arange(Lk) <= pos, 0.0, np.finfo(np.float16).min).astype(np.float16).reshape(1, 1, 1, Lk)
        mask = np.broadcast_to(mask, (B, 1, 1, Lk)).copy()
        a = _check(ctx, q, k, v, bias=mask, scale=1.0, expect="RowsSDPAPlan", what=f"mask pos {pos}")
        b = _check(ctx, q, k, v, kv_len=[pos + 1] * B, scale=1.0, expect="RowsSDPAPlan", what=f"kv_len pos {pos}")
        np.testing.assert_allclose(a.astype(np.float32), b.astype(np.float32), rtol=2e-3, atol=2e-3)


def test_full_bias_f32(ctx):
    B, H, Lq, Lk, E = 1, 2, 70, 90, 64
    q, k, v = _qkv(B, H, Lq, Lk, E, 81)
    bias = oracle.randn_f32((B, H, Lq, Lk), 84)
    _check(ctx, q, k, v, bias=bias, expect="FlashPlan", what="full f32 bias")
    _check(ctx, q[:, :, :40], k, v, bias=bias[:, :, :40].copy(), expect="RowsSDPAPlan", what="full f32 bias, 40 query rows")


@pytest.mark.parametrize("B,H,Lq,Lk,E,kind", [
    (2, 3, 200, 136, 64, "pad16"),        # (B,1,1,Lk) fp16 0 / finfo.min padding mask, broadcast over heads and queries
    (1, 2, 130, 260, 64, "full16"),       # dense fp16 (B,H,Lq,Lk), ragged last key block (260 = 4 x 64 + 4)
    (1, 2, 300, 333, 64, "full32"),       # dense fp32, an odd row length (fp32 rows are always dword aligned)
    (2, 2, 128, 130, 72, "causal16"),     # 0 / -inf lower-triangular mask (Lq, Lk) broadcast over batch and heads, head size 72
    (1, 1, 192, 320, 128, "full32"),      # the 128-wide instance
    (1, 20, 1500, 1500, 64, "pad16"),     # config 2's attention with a padding mask: an fp16 mask on a grid of at most one workgroup
    (2, 4, 300, 700, 64, "causal16"),     # per CU over 256 keys or more rides in the eight-wave key-halves form (so does full16 above)
    (3, 2, 150, 450, 64, "full16"),       # ... second half of the last stage with two keys
])
def test_additive_mask_rides_in_the_fused_kernel(ctx, B, H, Lq, Lk, E, kind):
    """Encoder-sized attention with an additive mask: the mask tile joins the scores inside the fused kernel (the
    reference's own fused plan declines masks, flash.jl:1327, and falls to its three-pass form, attention.jl:55-59)."""
    q, k, v = _qkv(B, H, Lq, Lk, E, 87)
    if kind == "pad16":
        valid = [Lk - 7 * (b + 1) for b in range(B)]
        bias = np.zeros((B, 1, 1, Lk), dtype=np.float16)
        for b in range(B):
            bias[b, :, :, valid[b]:] = np.finfo(np.float16).min
    elif kind == "full16":
        bias = oracle.randn_f16((B, H, Lq, Lk), 88)
    elif kind == "full32":
        bias = oracle.randn_f32((B, H, Lq, Lk), 89)
    else:
        bias = np.where(np.arange(Lk)[None, :] <= np.arange(Lq)[:, None] + (Lk - Lq), 0.0, -np.inf).astype(np.float16).reshape(1, 1, Lq, Lk)
    got = _check(ctx, q, k, v, bias=bias, expect="FlashPlan", what=f"fused mask {kind} {B},{H},{Lq},{Lk},{E}")
    if kind == "pad16":       # the same thing said with kv_len
        other = _check(ctx, q, k, v, kv_len=valid, expect="FlashPlan", what="kv_len twin")
        np.testing.assert_allclose(got.astype(np.float32), other.astype(np.float32), rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("B,H,Lq,Lk,E,kind", [
    (2, 3, 200, 136, 64, "values"),       # (B,1,1,Lk): random finite values, four-wave form, a ragged last block
    (2, 3, 200, 333, 64, "holes"),        # 0 / -inf with masked keys anywhere, not only at the end; odd row length
    (1, 20, 1500, 1500, 64, "holes"),     # config 2's grid: the eight-wave key-halves form
    (2, 4, 300, 700, 64, "perhead"),      # (B,H,1,Lk): a different key bias per head, key-halves form
    (3, 2, 150, 450, 64, "values"),       # key-halves form, second half of the last stage with two keys
    (2, 2, 128, 130, 72, "holes"),        # the 96-wide instance
    (1, 2, 192, 320, 128, "perhead"),     # the 128-wide instance
    (1, 2, 128, 64, 64, "allmasked"),     # every key -inf: zeros, as kv_len = 0 gives
    (2, 48, 1024, 1024, 64, "holes"),     # a grid large enough for the 256-query ping-pong form
    (3, 40, 700, 333, 64, "values"),      # ... ragged in queries and keys
    (1, 1, 128, 4096, 64, "holes"),       # the longest row that is kept in LDS
    (1, 1, 128, 4160, 64, "holes"),       # longer ones are read like any other mask
])
def test_key_only_mask_enters_with_the_first_product(ctx, B, H, Lq, Lk, E, kind):
    """An fp16 mask that is the same for every query -- a padding mask (B,1,1,Lk), a per-head key bias (B,H,1,Lk) -- is
    added by the first product's extra k-step, not by vector instructions: held to the same oracle as the dense mask,
    and to the dense-mask kernel's own result on the mask written out per query."""
    q, k, v = _qkv(B, H, Lq, Lk, E, 187)
    rng = np.random.default_rng(188)
    Hm = H if kind == "perhead" else 1
    if kind in ("values", "perhead"):
        bias = (rng.standard_normal((B, Hm, 1, Lk)) * 3).astype(np.float16)
    elif kind == "holes":
        bias = np.where(rng.random((B, Hm, 1, Lk)) < 0.3, -np.inf, 0.0).astype(np.float16)
        bias[..., 0] = 0.0                                             # at least one key stays
    else:
        bias = np.full((B, Hm, 1, Lk), -np.inf, dtype=np.float16)
    got = _check(ctx, q, k, v, bias=bias, expect="FlashPlan", what=f"key-only mask {kind} {B},{H},{Lq},{Lk},{E}")
    if kind == "allmasked":
        assert np.all(got == 0)
        return
    dense = np.ascontiguousarray(np.broadcast_to(bias, (B, H, Lq, Lk)))
    other = _check(ctx, q, k, v, bias=dense, what="the same mask written out per query")
    np.testing.assert_allclose(got.astype(np.float32), other.astype(np.float32), rtol=2e-3, atol=2e-3)


def test_mask_the_fused_kernel_cannot_read_takes_the_rows_kernel(ctx):
    q, k, v = _qkv(1, 2, 128, 129, 64, 90)
    bias = oracle.randn_f16((1, 2, 128, 129), 91)                     # fp16 rows of 129: every other row at a 2-byte offset
    _check(ctx, q, k, v, bias=bias, expect="RowsSDPAPlan", what="odd fp16 rows")
    import torch
    bt = to_dev(oracle.randn_f16((1, 2, 136, 128), 92)).transpose(2, 3)      # (B,H,Lq=128,Lk=136) with the queries contiguous
    _check(ctx, q[:, :, :, :], oracle.randn_f16((1, 2, 136, 64), 93), oracle.randn_f16((1, 2, 136, 64), 94), bias=None, what="sanity")
    assert type(__import__("juliavision_amd").sdpaplan(ctx, to_dev(q), to_dev(oracle.randn_f16((1, 2, 136, 64), 93)), to_dev(oracle.randn_f16((1, 2, 136, 64), 94)), bt)).__name__ == "RowsSDPAPlan"


def test_all_masked_rows_give_zeros(ctx):
    import torch
    B, H, Lq, Lk, E = 2, 2, 128, 64, 64
    q, k, v = _qkv(B, H, Lq, Lk, E, 91)
    got = _check(ctx, q, k, v, kv_len=[0, 40], expect="FlashPlan", what="kv_len 0 flash")
    assert np.all(got[0] == 0)
    q1 = q[:, :, :1]
    got = _check(ctx, q1, k, v, kv_len=[0, 40], expect="RowsSDPAPlan", what="kv_len 0 rows")
    assert np.all(got[0] == 0)
    mask = np.full((B, 1, 1, Lk), -np.inf, dtype=np.float32)
    got = _check(ctx, q1, k, v, bias=mask, what="-inf mask")
    assert np.all(got == 0)


def test_rows_sum_to_one(ctx):
    """softmax weights sum to 1: with v == 1 the output is exactly 1 up to fp16 rounding."""
    import torch
    B, H, Lq, Lk, E = 1, 2, 200, 333, 64
    q, k, _ = _qkv(B, H, Lq, Lk, E, 95)
    v = np.ones((B, H, Lk, E), dtype=np.float16)
    got = _check(ctx, q, k, v, what="v=1")
    assert np.max(np.abs(got.astype(np.float32) - 1.0)) < 2e-3


def test_config4_attention_full(ctx):
    """BASELINE config 4 attention at full size (L=4096, 16 heads x 64) against the oracle's composed fp32 form on every
    query row of every head (0.4 s of CPU per head), head by head so that one bad head cannot hide in the average."""
    import torch
    import juliavision_amd as jv
    B, H, L, E = 1, 16, 4096, 64
    q, k, v = _qkv(B, H, L, L, E, 101)
    out = poison(torch.empty((B, H, L, E), dtype=torch.float16, device="cuda"))
    jv.sdpa(ctx, to_dev(q), to_dev(k), to_dev(v), None, None, out=out)
    torch.cuda.synchronize()
    got = to_host(out)
    assert np.all(np.isfinite(got))
    for h in range(H):
        want = oracle.sdpa_ref_f32(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1])
        assert_parity(got[:, h:h + 1], want, what=f"config4 head {h}")


def test_token_major_output(ctx):
    """out given as a strided view: the result lands token-major ([B][L][H][E]), the layout the graph's
    permute + reshape after attention produces, with no copy."""
    import torch
    import juliavision_amd as jv
    B, H, L, E = 1, 4, 300, 64
    q, k, v = _qkv(B, H, L, L, E, 111)
    for lq in (L, 3):
        buf = poison(torch.empty((B, lq, H, E), dtype=torch.float16, device="cuda"))
        out = buf.permute(0, 2, 1, 3)
        ctx.ws.reset()
        jv.sdpa(ctx, to_dev(q[:, :, :lq]), to_dev(k), to_dev(v), None, None, out=out)
        torch.cuda.synchronize()
        want = oracle.sdpa_ref_f32(q[:, :, :lq], k, v)
        assert_parity(to_host(buf).transpose(0, 2, 1, 3), want, what=f"token-major out Lq={lq}")


def test_eight_wave_kernel_on_large_grids(ctx):
    """Grids that fill the chip with 256-query workgroups take the 8-wave variant of the fused kernel:
    ragged query and key counts, per-batch kv_len (one of them 0), strided heads."""
    import torch
    B, H, Lq, Lk, E = 4, 16, 700, 777, 64
    q, k, v = _qkv(B, H, Lq, Lk, E, 121)
    _check(ctx, q, k, v, expect="FlashPlan", what="8-wave ragged")
    got = _check(ctx, q, k, v, kv_len=[777, 0, 65, 300], expect="FlashPlan", what="8-wave kv_len")
    assert np.all(got[1] == 0)
    _check(ctx, q, k[:, :, :64], v[:, :, :64], expect="FlashPlan", what="8-wave one block")
    _check(ctx, q, k[:, :, :129], v[:, :, :129], out_dtype="f32", expect="FlashPlan", what="8-wave three blocks f32")


@pytest.mark.parametrize("Lk", [256, 257, 319, 320, 321, 383, 384, 385, 449, 1000])
def test_eight_wave_kernel_key_counts_around_block_boundaries(ctx, Lk):
    """256-query workgroups that cover the chip: key counts around the 64- and 128-key boundaries, a ragged last query
    block, per-batch lengths (0, below one block, a block short of the end), fp32 output."""
    q, k, v = _qkv(4, 16, 700, Lk, 64, 9000 + Lk, std=1.3)
    _check(ctx, q, k, v, expect="FlashPlan", what=f"8-wave Lk{Lk}")
    got = _check(ctx, q, k, v, kv_len=[Lk, 0, 37, Lk - 60], out_dtype="f32", expect="FlashPlan", what=f"8-wave kv_len Lk{Lk}")
    assert np.all(got[1] == 0)


@pytest.mark.parametrize("B,H,Lq,Lk,E", [(4, 16, 768, 65, 64), (4, 12, 1024, 257, 32), (2, 48, 520, 129, 64),
                                         (4, 16, 768, 1, 64), (3, 22, 770, 300, 48)])
def test_eight_wave_kernel_odd_key_counts_and_random_lengths(ctx, B, H, Lq, Lk, E):
    """The 8-wave variant alternates its two groups between a vector half and a matrix half, the next block's
    scores being formed one half ahead: key counts that end inside, on and one past a block, a single key, a
    head size below 64 and per-batch lengths drawn at random (0 and Lk included by the seed) must not show."""
    q, k, v = _qkv(B, H, Lq, Lk, E, 7000 + Lk, std=1.5)
    _check(ctx, q, k, v, expect="FlashPlan", what="8-wave odd keys")
    lens = np.random.default_rng(Lk).integers(0, Lk + 1, size=B)
    lens[0], lens[-1] = Lk, 0
    got = _check(ctx, q, k, v, kv_len=[int(x) for x in lens], expect="FlashPlan", what="8-wave random kv_len")
    assert np.all(got[-1] == 0)


def test_fused_kernel_splits_keys_on_small_grids(ctx):
    """Few query blocks and very many keys: the fused kernel also splits the keys over workgroups and a merge joins
    the partials.  Ragged last split, per-batch kv_len that leaves the later split without a key (one row of the
    batch with none at all), fp32 and token-major outputs; config 3's shape stays in one pass.  Head size 48 here: at
    64 these extents run the short-chain form, which splits the keys inside the workgroup."""
    import torch
    import juliavision_amd as jv
    q, k, v = _qkv(1, 6, 1370, 1370, 64, 131)
    plan = jv.sdpaplan(ctx, to_dev(q), to_dev(k), to_dev(v))
    assert type(plan).__name__ == "FlashPlan" and plan.nsplit == 1, plan
    _check(ctx, q, k, v, expect="FlashPlan", what="config 3 attention")
    q, k, v = _qkv(1, 2, 300, 2000, 48, 135)
    assert jv.sdpaplan(ctx, to_dev(q), to_dev(k), to_dev(v)).nsplit == 2
    _check(ctx, q, k, v, expect="FlashPlan", what="two key splits, ragged second")
    q, k, v = _qkv(3, 2, 200, 1700, 48, 141)
    assert jv.sdpaplan(ctx, to_dev(q), to_dev(k), to_dev(v)).nsplit == 2
    got = _check(ctx, q, k, v, kv_len=[1700, 0, 70], out_dtype="f32", expect="FlashPlan", what="key splits with kv_len")
    assert np.all(got[1] == 0)
    buf = poison(torch.empty((3, 200, 2, 48), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.sdpa(ctx, to_dev(q), to_dev(k), to_dev(v), None, None, out=buf.permute(0, 2, 1, 3))
    torch.cuda.synchronize()
    assert_parity(to_host(buf).transpose(0, 2, 1, 3), oracle.sdpa_ref_f32(q, k, v), what="key splits, token-major out")
    # without a workspace the same call runs unsplit and must agree
    from juliavision_amd import _lib as L
    lib = L.init()
    dq, dk, dv = to_dev(q), to_dev(k), to_dev(v)
    out = poison(torch.empty((3, 2, 200, 48), dtype=torch.float16, device="cuda"))
    st = lambda t: L.strides4(t.stride(3), t.stride(2), t.stride(1), t.stride(0))
    rc = lib.mi_sdpa_f16(out.data_ptr(), L.F16, None, dq.data_ptr(), st(dq), dk.data_ptr(), st(dk), dv.data_ptr(), st(dv),
                         None, L.F16, None, None, 48, 200, 1700, 2, 3, 48 ** -0.5, None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert_parity(to_host(out), oracle.sdpa_ref_f32(q, k, v), what="no workspace: one pass")


@pytest.mark.parametrize("Lk", [256, 257, 319, 320, 321, 383, 384, 385, 447, 448, 449, 1000])
@pytest.mark.parametrize("B,H,Lq,E", [(5, 20, 256, 64), (4, 20, 300, 64), (2, 3, 200, 32)])
def test_fused_kernel_key_halves_on_one_workgroup_per_cu_grids(ctx, B, H, Lq, Lk, E):
    """Grids of at most one 128-query workgroup per CU with 256 keys or more (and, at head size 64, more 64-query tiles
    than CUs: 400 and 400 here) run eight waves, each pair of waves sharing its queries and taking alternate 64-key
    halves of a 128-key stage; the halves merge in LDS.  Key counts around the 64- and 128-key boundaries: the second
    half's last block empty, ragged, exactly full."""
    q, k, v = _qkv(B, H, Lq, Lk, E, 211 + Lk)
    _check(ctx, q, k, v, expect="FlashPlan", what=f"key halves B{B} H{H} Lq{Lq} Lk{Lk} E{E}")


@pytest.mark.parametrize("Lk", [128, 129, 255, 256, 257, 300, 511, 512, 513, 767, 768, 769, 1000, 1370])
@pytest.mark.parametrize("B,H,Lq", [(2, 3, 64), (1, 6, 130), (1, 2, 1370)])
def test_short_chain_form_on_small_grids(ctx, B, H, Lq, Lk):
    """Head size 64 and at most about one 32-query tile per CU: four waves per tile, each walking its own quarter of the
    keys (whole 64-key blocks), K fragments straight from memory, partials merged in LDS.  Key counts around the
    boundaries of a wave's share: waves without a key, with a ragged block, with exactly full ones; a ragged last tile
    of queries."""
    q, k, v = _qkv(B, H, Lq, Lk, 64, 411 + Lk)
    _check(ctx, q, k, v, expect="FlashPlan", what=f"short chain B{B} H{H} Lq{Lq} Lk{Lk}")


@pytest.mark.parametrize("Lk", [128, 129, 191, 192, 193, 255, 256, 257, 300, 511, 512, 513, 769, 1000, 1370])
@pytest.mark.parametrize("B,H,Lq", [(12, 12, 64), (5, 12, 130), (1, 6, 1370), (3, 40, 65)])
def test_pair_form_where_64_query_tiles_fit_the_cus(ctx, B, H, Lq, Lk):
    """Head size 64, more 32-query tiles than CUs, at most one 64-query tile per CU: eight waves per tile, wave w on key
    quarter w % 4 for query half w / 4, the two waves of a quarter sharing its K and V through LDS.  Key counts around
    the boundaries of a quarter's share (quarters without a key, with a ragged block, with exactly full ones); tiles
    whose second query half is ragged (130, 1370) or a single query (65)."""
    q, k, v = _qkv(B, H, Lq, Lk, 64, 511 + Lk)
    _check(ctx, q, k, v, expect="FlashPlan", what=f"pair form B{B} H{H} Lq{Lq} Lk{Lk}")


@pytest.mark.parametrize("H,HP", [(2, 6), (10, 32), (20, 64)])
def test_fused_kernel_key_halves_masks_and_layouts(ctx, H, HP):
    """H = 2, HP = 6: the short-chain form (60 and 54 tiles of 32 queries); H = 10, HP = 32: the pair form (300 and 288
    tiles of 32, 180 and 160 of 64); H = 20, HP = 64: the key-halves form (360 and 320 tiles of 64, 240 and 192 of 128)."""
    import torch
    import juliavision_amd as jv
    q, k, v = _qkv(6, H, 150, 300, 64, 251)
    # kv_len leaves the second half of the keys without a valid one (10, 64), with exactly one (65), a ragged
    # second stage (129, 200), and a row of the batch with none at all (0)
    got = _check(ctx, q, k, v, kv_len=[10, 64, 65, 129, 0, 200], out_dtype="f32", expect="FlashPlan", what="key halves with kv_len")
    assert np.all(got[4] == 0)
    # large scores: the reference point has to move in one half and not the other
    q2 = q.copy()
    q2[:, :, :, :] *= np.float16(6.0)
    k2 = k.copy()
    k2[:, :, 64:128] *= np.float16(3.0)
    _check(ctx, q2, k2, v, expect="FlashPlan", what="key halves, one half with far larger scores")
    # token-major output and packed strided q/k/v, as the encoder block calls it
    B, H, L, E = 1, HP, 260, 64
    qkv = oracle.randn_f16((L, 3 * H * E), 261)
    dqkv = to_dev(qkv)
    views = [dqkv[:, i * H * E:(i + 1) * H * E].unflatten(1, (H, E)).permute(1, 0, 2).unsqueeze(0) for i in range(3)]
    buf = poison(torch.empty((L, H * E), dtype=torch.float16, device="cuda"))
    ctx.ws.reset()
    jv.sdpa(ctx, *views, None, None, out=buf.unflatten(1, (H, E)).permute(1, 0, 2).unsqueeze(0))
    torch.cuda.synchronize()
    hq, hk, hv = (np.ascontiguousarray(qkv[:, i * H * E:(i + 1) * H * E].reshape(L, H, E).transpose(1, 0, 2))[None] for i in range(3))
    want = oracle.sdpa_ref_f32(hq, hk, hv)
    assert_parity(to_host(buf).reshape(L, H, E).transpose(1, 0, 2)[None], want, what="key halves, token-major")


@pytest.mark.parametrize("B,H,Lq,Lk,which", [(1, 2, 128, 200, "four waves"), (4, 16, 300, 200, "eight waves, 256 queries"),
                                             (1, 3, 128, 400, "short chain"), (8, 12, 128, 400, "key halves"), (1, 2, 200, 8000, "key splits"),
                                             (4, 24, 300, 400, "eight waves, 256 queries, 400 keys")])
def test_reference_point_follows_scores_that_grow_along_the_keys(ctx, B, H, Lq, Lk, which):
    """The fused kernel exponentiates against a reference point that it moves only when it must.  Keys whose scores
    exceed everything before them by far more than fp16's exponent range (here by up to ~2^60 from one 64-key block
    to a later one, for some queries and not for others) must move it; attention then is nearly one-hot on them."""
    q, k, v = _qkv(B, H, Lq, Lk, 64, 301)
    q = (q.astype(np.float32) * 3.0).astype(np.float16)
    k = k.copy()
    k[:, :, 70:75] *= np.float16(4.0)            # second block
    k[:, :, 150:152] *= np.float16(8.0)          # third block: dominates for the queries aligned with it
    if Lk > 330:
        k[:, :, 330] *= np.float16(10.0)
    got = _check(ctx, q, k, v, expect="FlashPlan", what=f"growing scores, {which}")
    assert np.all(np.isfinite(got))


@pytest.mark.parametrize("Lk", [1, 7, 8, 63, 64, 65, 383, 384, 385, 448, 640, 1500, 4097])
@pytest.mark.parametrize("E", [64, 40, 16])
def test_single_query_over_a_short_key_range_runs_in_one_launch(ctx, Lk, E):
    """Lq = 1 (a decode step): one launch, eight-wave workgroups striding the keys in rounds of six passes, the key
    range beyond 512 keys cut over several workgroups (a round of six passes each) that merge inside the launch.
    Key counts around the pass (64) and round (384) sizes, and ranges that split 2, 4 and 11 ways."""
    import juliavision_amd as jv
    q, k, v = _qkv(3, 5, 1, Lk, E, 401 + Lk)
    plan = jv.sdpaplan(ctx, to_dev(q), to_dev(k), to_dev(v))
    passes = (Lk + 63) // 64
    want = 1 if passes <= 8 else max(1, min(ctx.dev.cores // 15, -(-passes // 6)))
    while want > 1 and -(-((Lk + 63) // 64) // want) * (want - 1) >= (Lk + 63) // 64:
        want -= 1
    assert type(plan).__name__ == "RowsSDPAPlan" and plan.nsplit == want, plan
    _check(ctx, q, k, v, expect="RowsSDPAPlan", what=f"one-launch decode attention Lk{Lk} E{E}")
    lens = [Lk, 0, max(1, Lk // 2)]
    got = _check(ctx, q, k, v, kv_len=lens, out_dtype="f32", expect="RowsSDPAPlan", what=f"one-launch decode attention Lk{Lk} E{E} kv_len")
    assert np.all(got[1] == 0)
