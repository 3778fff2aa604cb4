"""The unfused permute path of the reference (expert_permute.py:43-68):
expert_input_permute = routing preprocessing + row gather, expert_output_permute = row scatter
+ top-k combine.  Bit-exact against the oracle's routing and plain indexing; the round trip
permute -> (identity experts) -> un-permute must give sum_j scores[t, j] * x[t]."""
import pytest
import torch

from oracle import moe_ref
from util import assert_parity, randn, seeded

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,d,E,k,dtype", [
    (128, 128, 8, 2, torch.bfloat16), (999, 256, 64, 8, torch.float16), (5, 64, 8, 2, torch.float32),
    (2011, 2048, 64, 8, torch.bfloat16), (300, 100, 16, 3, torch.float32),
])
def test_expert_input_permute(T, d, E, k, dtype):
    from moe_explore.expert_permute import GroupedTokens, expert_input_permute
    g = seeded(T + d)
    x = randn((T, d), g, dtype)
    _, idx = moe_ref.route_from_logits(torch.randn((T, E), generator=g), k, True, False, dtype)
    gt = expert_input_permute(x.cuda(), idx.cuda(), E, k)
    assert isinstance(gt, GroupedTokens)
    gi, ind = moe_ref.get_token_indices(idx, k, E, zero_prefix=True)
    assert gt.group_indices.dtype == torch.int32 and gt.indices.dtype == torch.int64
    assert torch.equal(gt.group_indices.cpu(), gi)
    assert torch.equal(gt.indices.cpu(), ind)
    assert gt.tokens.shape == (T * k, d) and gt.tokens.dtype == dtype
    assert torch.equal(gt.tokens.cpu(), x[ind // k])          # a copy: exact
    # rows of expert e are the tokens routed to e
    flat = idx.reshape(-1)
    for e in range(E):
        lo, hi = int(gi[e]), int(gi[e + 1])
        assert (flat[ind[lo:hi]] == e).all()


@pytest.mark.parametrize("T,d,E,k,dtype", [
    (128, 128, 8, 2, torch.bfloat16), (999, 256, 64, 8, torch.float16), (77, 72, 8, 2, torch.float32),
    (2011, 1024, 64, 8, torch.bfloat16),
])
def test_permute_round_trip(T, d, E, k, dtype):
    """expert_output_permute(expert_input_permute(x)) with nothing in between is
    out[t] = sum_j scores[t, j] * x[t]; with a per-expert scaling of the grouped rows in between
    it is the layer with 'experts' y = c_e * x, against the oracle's combine."""
    from moe_explore.expert_permute import GroupedTokens, expert_input_permute, expert_output_permute
    g = seeded(T * 3 + d)
    x = randn((T, d), g, dtype)
    scores, idx = moe_ref.route_from_logits(torch.randn((T, E), generator=g), k, True, True, dtype)
    gt = expert_input_permute(x.cuda(), idx.cuda(), E, k)
    out = expert_output_permute(gt, scores.cuda(), k, x.shape)
    assert out.shape == x.shape and out.dtype == dtype
    want = x.float() * scores.float().sum(-1, keepdim=True)
    assert_parity(out, want, dtype, "identity round trip", tol=1e-5 if dtype == torch.float32 else 2e-2)
    # per-expert scale c_e = e + 1 applied to the grouped rows (exact in every dtype for small e)
    gi = gt.group_indices.cpu()
    scale = torch.repeat_interleave(torch.arange(1, E + 1, dtype=torch.float32), (gi[1:] - gi[:-1]).long())
    scaled = (gt.tokens.float() * scale.cuda().unsqueeze(1)).to(dtype)
    out2 = expert_output_permute(GroupedTokens(scaled, gt.group_indices, gt.indices), scores.cuda(), k, x.shape)
    y_slots = (x.float().unsqueeze(1) * (idx.float() + 1.0).unsqueeze(-1)).to(dtype).float()   # [T, k, d]
    want2 = moe_ref.scale_and_reduce(y_slots.reshape(T * k, d), scores.float(), T, k)
    assert_parity(out2, want2, dtype, "scaled round trip", tol=1e-5 if dtype == torch.float32 else 2e-2)
