"""Committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py
from the pinned oracle): the oracle must still reproduce them on the CPU, and the HIP
path must reproduce them on the GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import moe_ref

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return {k: torch.from_numpy(v) for k, v in np.load(os.path.join(GOLD, name)).items()}


def test_oracle_reproduces_routing_vector():
    f = load("routing_r200_e8.npz")
    gi, idx = moe_ref.get_token_indices(f["expert_ids"], 1, 8, zero_prefix=True)
    assert torch.equal(gi, f["group_indices"]) and torch.equal(idx, f["indices"])
    assert (f["group_indices"][8] == f["group_indices"][7])  # the empty expert


def test_oracle_reproduces_layer_vector():
    f = load("layer_t48_d32_ff24_e4_top2_swiglu_fp32.npz")
    out, dx, dw1, dw2, ds = moe_ref.experts_backward(f["x"], f["w1"], f["w2"], f["scores"],
                                                     f["expert_ids"], 4, 2, "swiglu", f["dout"])
    for got, key in ((out, "out"), (dx, "dx"), (dw1, "dw1"), (dw2, "dw2"), (ds, "dscores")):
        torch.testing.assert_close(got, f[key], rtol=1e-5, atol=1e-6)


def test_oracle_reproduces_grouped_gemm_vector():
    f = load("grouped_gemm_t40_e4_top2_k16_n24_fp32.npz")
    g = moe_ref.grouped_matmul_gather_scatter(f["a"], f["w"], f["group_indices"], f["indices"],
                                              gather=True, topk=2, activation_name="geglu")
    torch.testing.assert_close(g, f["gathered_geglu"], rtol=1e-5, atol=1e-6)
    c = moe_ref.grouped_matmul_gather_scatter(f["rows"], f["w"], f["group_indices"], f["indices"],
                                              scatter=True, num_tokens=40, topk=2, scales=f["scores"])
    torch.testing.assert_close(c, f["combined"], rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_hip_routing_vector():
    from moe_explore.expert_permute import get_token_indices
    f = load("routing_r200_e8.npz")
    p = get_token_indices(f["expert_ids"].cuda(), 1, 8, zero_prefix=True)
    assert torch.equal(p.group_indices.cpu(), f["group_indices"])
    assert torch.equal(p.indices.cpu(), f["indices"])


@pytest.mark.gpu
def test_hip_layer_vector():
    from moe_explore.functional.topk_moe import routed_experts
    f = load("layer_t48_d32_ff24_e4_top2_swiglu_fp32.npz")
    x, w1, w2, sc = (f[k].cuda().requires_grad_(True) for k in ("x", "w1", "w2", "scores"))
    out = routed_experts(x, w1, w2, sc, f["expert_ids"].cuda(), 4, 2, "swiglu")
    out.backward(f["dout"].cuda())
    for got, key in ((out, "out"), (x.grad, "dx"), (w1.grad, "dw1"), (w2.grad, "dw2"),
                     (sc.grad, "dscores")):
        assert moe_ref.rel_fro(got, f[key]) <= 1e-5, key
        assert moe_ref.rel_max(got, f[key]) <= 1e-5, key


@pytest.mark.gpu
def test_hip_grouped_gemm_vector():
    from moe_explore.triton_kernels.m_grouped_gemm import MGroupedGEMMParams, m_grouped_gemm
    from moe_explore.functional.scale_and_reduce import scale_and_reduce
    f = load("grouped_gemm_t40_e4_top2_k16_n24_fp32.npz")
    gi, perm, w = f["group_indices"].cuda(), f["indices"].cuda(), f["w"].cuda()
    g = m_grouped_gemm(f["a"].cuda(), MGroupedGEMMParams(w, gi, perm, True, False, 40, 2, activation="geglu"))
    assert moe_ref.rel_max(g, f["gathered_geglu"]) <= 1e-5
    p = MGroupedGEMMParams(w, gi, perm, False, True, 40, 2, scales=f["scores"].cuda())
    y = m_grouped_gemm(f["rows"].cuda(), p)
    c = scale_and_reduce(y, p.scales, 40, 2, y.size(1))
    assert moe_ref.rel_max(c, f["combined"]) <= 1e-5
    fused = m_grouped_gemm(f["rows"].cuda(), p, combine=True)
    assert moe_ref.rel_max(fused, f["combined"]) <= 1e-5
