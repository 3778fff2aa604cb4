"""Smoke run of the grouped-GEMM sweep (the counterpart of the reference's
bench/bench_m_grouped_gemm.py): one small row per routing kind, the CSV layout, and the OLMoE
load table's routing generator."""
import csv
import importlib.util
import math
import os

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _sweep_module():
    spec = importlib.util.spec_from_file_location(
        "bench_m_grouped_gemm", os.path.join(ROOT, "moe-explore_amd", "bench_m_grouped_gemm.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_olmoe_routing_follows_the_load_table():
    from moe_explore.testing import OLMOE_EXPERT_LOAD_PERCENT, random_olmoe_routing
    torch.manual_seed(0)
    T, E, k = 20000, 64, 8
    scores, idx = random_olmoe_routing(T, E, k, "cpu", torch.bfloat16)
    assert scores.shape == (T, k) and idx.shape == (T, k) and scores.dtype == torch.bfloat16
    assert (torch.sort(idx, -1).values.diff(dim=-1) > 0).all(), "an expert chosen twice for a token"
    load = torch.bincount(idx.flatten(), minlength=E).float() / T * 100.0
    table = torch.tensor(OLMOE_EXPERT_LOAD_PERCENT)
    assert abs(sum(OLMOE_EXPERT_LOAD_PERCENT) - 800.0) < 1.0       # top-8: the shares sum to 8
    # sampling without replacement flattens the heaviest experts a little; the ranking stays
    assert torch.corrcoef(torch.stack((load, table)))[0, 1] > 0.98
    assert load.argmax() == table.argmax() and load[table.argmin()] < 4.0


@pytest.mark.gpu
@pytest.mark.parametrize("routing", ["balanced", "skewed", "olmoe", "perfect"])
def test_one_row_of_the_sweep(routing, tmp_path):
    mod = _sweep_module()
    rows = mod.run_sweep("olmoe", routing, [512], warmup=1, reps=3)
    assert len(rows) == 1 and rows[0]["num_tokens"] == 512
    for name in mod.PROVIDERS:
        v = rows[0][name]
        assert math.isnan(v) and name == "gemm-reference" or (v > 0 and math.isfinite(v)), name
    path = tmp_path / "sweep.csv"
    mod.write_csv(rows, path)
    with open(path) as f:
        got = list(csv.reader(f))
    assert got[0] == ["num_tokens", *mod.PROVIDERS] and got[1][0] == "512" and len(got[1]) == 5
