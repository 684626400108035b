"""The committed vectors of tests/golden/path_vectors.npz (made by tests/golden/make_golden.py from the closed-form
inputs of the reference's own tests): on the CPU, the oracle must still return what was frozen and that must agree
with the independent float64 closed form stored beside it; on the GPU, the HIP path must meet both."""
import os

import numpy as np
import pytest

import oracle
from util import assert_parity, poison, to_dev, to_host

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "path_vectors.npz"))
CASES = ["gemm", "gemm_gelu", "attn", "attn72", "conv3", "conv5", "convt", "ln"]


def _oracle_run(case):
    if case in ("gemm", "gemm_gelu"):
        return oracle.gemm_f16(G["gemm_x"], G["gemm_w"], G["gemm_bias"], epi="gelu" if case == "gemm_gelu" else "none")
    if case in ("attn", "attn72"):
        kl = G[case + "_kv_len"] if case + "_kv_len" in G else None
        return oracle.sdpa_threepass_f16(G[case + "_q"], G[case + "_k"], G[case + "_v"], kv_len=kl)
    if case in ("conv3", "conv5"):
        s, p = (int(v) for v in G[case + "_geom"])
        return oracle.conv2d_f16(G[case + "_x"], G[case + "_w"], G[case + "_bias"], (s, s), (p, p))
    if case == "convt":
        return oracle.convtranspose2d_f16(G["convt_x"], G["convt_w"], G["convt_bias"], (2, 2))
    return oracle.layernorm_f16(G["ln_a"], G["ln_gamma"], G["ln_beta"], eps=1e-6)[0]


@pytest.mark.parametrize("case", CASES)
def test_oracle_returns_the_frozen_vectors(case):
    got = _oracle_run(case)
    assert got.dtype == np.float16
    assert np.array_equal(got.view(np.uint16), G[case + "_oracle"].view(np.uint16)), f"{case}: the oracle's output changed"


@pytest.mark.parametrize("case", CASES)
def test_frozen_vectors_meet_the_float64_closed_form(case):
    # one fp16 rounding of a sum accumulated in fp32: well inside 2e-3 of the largest value
    assert_parity(G[case + "_oracle"], G[case + "_f64"], max_rel=2e-3, min_cos=0.999999, what=case)


def test_layernorm_statistics_of_the_frozen_vectors():
    a = G["ln_a"].astype(np.float64)
    assert np.allclose(G["ln_mean_oracle"], a.mean(axis=1), rtol=0, atol=1e-6)
    assert np.allclose(G["ln_rstd_oracle"], 1.0 / np.sqrt(a.var(axis=1) + 1e-6), rtol=1e-6)


def _hip_run(ctx, case):
    import torch
    import juliavision_amd as jv
    ctx.ws.reset()
    if case in ("gemm", "gemm_gelu"):
        x, w, b = to_dev(G["gemm_x"]), to_dev(G["gemm_w"]), to_dev(G["gemm_bias"])
        out = poison(torch.empty((x.shape[0], w.shape[1]), dtype=torch.float16, device="cuda"))
        return jv.matmul_(ctx, out, w, x, b, epi="gelu" if case == "gemm_gelu" else "none")
    if case in ("attn", "attn72"):
        q, k, v = (to_dev(G[case + n]) for n in ("_q", "_k", "_v"))
        kl = torch.from_numpy(G[case + "_kv_len"]).cuda() if case + "_kv_len" in G else None
        return jv.sdpa(ctx, q, k, v, out=poison(torch.empty_like(q)), kv_len=kl)
    if case in ("conv3", "conv5"):
        s, p = (int(v) for v in G[case + "_geom"])
        out = poison(torch.empty(G[case + "_oracle"].shape, dtype=torch.float16, device="cuda"))
        return jv.convolution_(ctx, out, to_dev(G[case + "_x"]), to_dev(G[case + "_w"]), to_dev(G[case + "_bias"]), (s, s), (p, p), (1, 1), 1)
    if case == "convt":
        out = poison(torch.empty(G["convt_oracle"].shape, dtype=torch.float16, device="cuda"))
        return jv.convolutiontranspose_(ctx, out, to_dev(G["convt_x"]), to_dev(G["convt_w"]), to_dev(G["convt_bias"]), (2, 2), (0, 0), (1, 1), (0, 0), 1)
    a = to_dev(G["ln_a"])
    return jv.layernorm_(ctx, poison(torch.empty_like(a)), None, None, a, to_dev(G["ln_gamma"]), to_dev(G["ln_beta"]), a.shape[1], 1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_hip_path_meets_the_golden_vectors(ctx, case):
    import torch
    got = _hip_run(ctx, case)
    torch.cuda.synchronize()
    got = to_host(got)
    assert_parity(got, G[case + "_oracle"], what=case + " vs the oracle's frozen output")
    assert_parity(got, G[case + "_f64"], what=case + " vs the float64 closed form")
