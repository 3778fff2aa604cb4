"""Test helpers of the reference (``testing.py``): the op-level PyTorch
comparison implementation, synthetic routing generators, weight initialisers and
the tolerance rule.  Plain PyTorch, any device; none of it is used by the HIP path."""
import math

import torch
import torch.nn.functional as F

from moe_explore.functional.activation import activation
from moe_explore.params import MLPParams, GLUParams, TopkRouterParams, ErnieRouterParams


def torch_grouped_matmul_gather_scatter(a, params):
    """Per-expert matmul with optional gather, scatter, activation and combine
    (``testing.py:9-50``).  All positions are gathered at once, every expert multiplies its
    slice of them, and the products are scattered at once."""
    weight, bounds = params.weight, params.group_indices.tolist()
    rows = a.index_select(0, params.permute_indices // params.topk) if params.gather else a
    products = [rows[lo:hi] @ weight[e] for e, (lo, hi) in enumerate(zip(bounds[:-1], bounds[1:]))]
    c = torch.cat(products) if products else rows.new_zeros((0, weight.size(-1)))
    if c.size(0) < rows.size(0):   # positions past the last group stay zero
        c = torch.cat([c, c.new_zeros((rows.size(0) - c.size(0), c.size(1)))])
    if params.scatter:
        c = torch.zeros_like(c).index_copy_(0, params.permute_indices.to(torch.int64), c)
    if params.activation is not None:
        c = activation(c, params.activation)
    if params.scatter and params.scales is not None:
        c = torch.einsum("tkn,tk->tn", c.view(params.num_tokens, params.topk, -1), params.scales.to(c.dtype))
    return c.to(a.dtype)


def torch_grouped_glu(a, params):
    """Grouped GLU with separate gate and up weights and an optional fused gather
    (``testing.py:52-85``): ``c[rows of group i] = act(a_i @ gate[i]) * (a_i @ up[i])``.
    ``params`` is any record with ``gate_weight``, ``up_weight`` ``[E, K, N]``,
    ``group_indices`` ``[E + 1]``, ``permute_indices``, ``gather``, ``topk`` and ``activation``
    ("silu" or "gelu", applied to the gate product)."""
    assert params.gate_weight.size() == params.up_weight.size()
    gather = bool(getattr(params, "gather", False))
    topk = getattr(params, "topk", 1)
    rows = params.permute_indices // topk if gather else None
    c = torch.zeros((a.size(0) * topk if gather else a.size(0), params.gate_weight.size(-1)),
                    device=a.device, dtype=a.dtype)
    bounds = params.group_indices.tolist()
    for i in range(params.gate_weight.size(0)):
        lo, hi = bounds[i], bounds[i + 1]
        a_i = a[rows[lo:hi]] if gather else a[lo:hi]
        c[lo:hi] = activation(a_i @ params.gate_weight[i], params.activation) * (a_i @ params.up_weight[i])
    return c


def perfect_routing(num_tokens, num_experts, topk, device, dtype):
    """Every expert gets the same number of rows (``testing.py:87-95``)."""
    assert num_tokens % num_experts == 0
    indices = torch.arange(0, num_tokens * topk, device=device) % num_experts
    topk_scores, _ = random_routing(num_tokens, num_experts, topk, device, dtype)
    return topk_scores, indices


def random_routing(num_tokens, num_experts, topk, device, dtype):
    """Top-k of a softmax over normal logits: near-uniform loads (``testing.py:97-106``)."""
    scores = F.softmax(torch.randn((num_tokens, num_experts), device=device, dtype=torch.float32), dim=-1)
    topk_logits, topk_indices = torch.topk(scores, k=topk, dim=-1, sorted=False)
    return topk_logits.to(dtype), topk_indices


def random_skewed_routing(num_tokens, num_experts, topk, num_skewed_experts, skew_factor, device, dtype):
    """``num_skewed_experts`` experts are ``skew_factor`` times likelier (``testing.py:108-132``)."""
    odds = torch.ones(num_experts, dtype=torch.float32)
    odds[torch.randperm(num_experts)[:num_skewed_experts]] = skew_factor
    topk_indices = torch.multinomial(odds.to(device).expand(num_tokens, num_experts), topk)
    return random_routing(num_tokens, num_experts, topk, device, dtype)[0], topk_indices


# Share (in percent, top-8) of tokens that reach each of OLMoE-1B-7B's 64 experts in the layer
# the reference measured (the table embedded in ``testing.py:141-206``, rounded to 1e-3).
OLMOE_EXPERT_LOAD_PERCENT = (
    18.016, 16.976, 12.5, 10.182, 7.372, 15.966, 9.168, 11.66, 15.418, 17.458, 10.972, 12.994,
    9.004, 17.926, 13.156, 10.016, 8.604, 21.036, 8.512, 3.96, 2.616, 6.664, 8.37, 16.756, 18.186,
    2.848, 7.324, 8.522, 9.532, 8.648, 12.092, 24.614, 15.37, 7.922, 13.118, 2.748, 16.314, 19.992,
    9.774, 13.298, 37.532, 16.268, 7.85, 12.164, 18.804, 10.76, 7.862, 19.14, 6.974, 13.958, 9.122,
    8.742, 12.018, 16.918, 26.756, 8.796, 4.726, 16.596, 7.27, 11.458, 9.91, 6.098, 26.756, 8.686,
)


def random_olmoe_routing(num_tokens, num_experts, topk, device, dtype):
    """Experts drawn without replacement with OLMoE's measured per-expert loads as weights
    (``testing.py:134-209``); 64 experts only, as there."""
    assert num_experts == len(OLMOE_EXPERT_LOAD_PERCENT), "the load table has 64 experts"
    probabilities = torch.tensor(OLMOE_EXPERT_LOAD_PERCENT, device=device, dtype=torch.float32) / 100.0
    topk_indices = torch.multinomial(probabilities.repeat(num_tokens, 1), num_samples=topk, replacement=False)
    topk_scores, _ = random_routing(num_tokens, num_experts, topk, device, dtype)
    return topk_scores, topk_indices


def random_zipf_routing(num_tokens, num_experts, topk, device, dtype, s=1.2, generator=None):
    """Top-k of normal logits plus ``log p_e`` with ``p_e`` Zipf(s) over a random
    permutation of the experts: a few heavy experts and some near-empty ones."""
    cpu_gen = generator
    ranks = torch.randperm(num_experts, generator=cpu_gen).to(torch.float32) + 1.0
    p = ranks.pow(-s)
    bias = torch.log(p / p.sum()).to(device)
    logits = torch.randn((num_tokens, num_experts), device=device, dtype=torch.float32) + bias
    scores = F.softmax(logits, dim=-1)
    topk_scores, topk_indices = torch.topk(scores, k=topk, dim=-1, sorted=False)
    topk_scores = topk_scores / topk_scores.sum(-1, keepdim=True)
    return topk_scores.to(dtype), topk_indices


def random_groups(num_tokens, num_groups, device):
    """``[0, r1 < r2 < ..., num_tokens]`` with random inner boundaries (``testing.py:212-224``)."""
    inner = torch.randperm(num_tokens - 2, device=device)[:num_groups - 1] + 1   # distinct, in 1 .. n-2
    ends = torch.tensor([0, num_tokens], device=device)
    return torch.cat([ends[:1], torch.sort(inner).values, ends[1:]]).to(torch.int32)


def uniform_weight_init(size, device, dtype):
    """Xavier-uniform-like initialisation (``testing.py:226-256``)."""
    weight = torch.empty(size, device=device, dtype=dtype)
    if len(size) == 1:
        return weight.uniform_(-0.02, 0.02)
    if len(size) == 2:
        torch.nn.init.xavier_uniform_(weight)
        return weight
    assert len(size) == 3
    a = math.sqrt(3) * math.sqrt(2 / (size[1] + size[2]))
    return weight.uniform_(-a, a)


def normal_weight_init(size, device, dtype):
    weight = torch.empty(size, device=device, dtype=dtype)
    torch.nn.init.normal_(weight, mean=0.0, std=0.02)
    return weight


def random_mlp(num_experts, hidden_dim, intermediate_dim, activation, device, dtype, dist=uniform_weight_init):
    return MLPParams(
        dist((num_experts, hidden_dim, intermediate_dim), device=device, dtype=dtype),
        dist((num_experts, intermediate_dim, hidden_dim), device=device, dtype=dtype),
        activation,
    )


def random_glu(num_experts, hidden_dim, intermediate_dim, activation, device, dtype, dist=uniform_weight_init):
    return GLUParams(
        dist((num_experts, hidden_dim, intermediate_dim), device=device, dtype=dtype),
        dist((num_experts, hidden_dim, intermediate_dim), device=device, dtype=dtype),
        dist((num_experts, intermediate_dim, hidden_dim), device=device, dtype=dtype),
        activation,
    )


def random_interleaved_glu(num_experts, hidden_dim, intermediate_dim, activation, device, dtype,
                           dist=uniform_weight_init):
    return MLPParams(
        dist((num_experts, hidden_dim, 2 * intermediate_dim), device=device, dtype=dtype),
        dist((num_experts, intermediate_dim, hidden_dim), device=device, dtype=dtype),
        activation,
    )


def random_topk_router(num_experts, hidden_dim, topk, softmax_before_topk, normalize_routing, device,
                       dtype, dist=uniform_weight_init):
    return TopkRouterParams(
        dist((hidden_dim, num_experts), device=device, dtype=dtype),
        topk,
        softmax_before_topk=softmax_before_topk,
        normalize_routing=normalize_routing,
    )


def random_ernie_router(num_experts, hidden_dim, topk, device, dtype, dist=uniform_weight_init):
    return ErnieRouterParams(
        dist((hidden_dim, num_experts), device=device, dtype=torch.float32),
        dist((num_experts,), device=device, dtype=torch.float32),
        topk,
    )


# one unit in the last place of 1.0 per dtype, as the reference's tolerance rule takes it
_EPS = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 1e-6}


def assert_close(a, b):
    """Tolerance rule of the reference's tests (``testing.py:340-357``): absolute tolerance
    ``min(1e-2, k * max * eps / 100)``, relative ``sqrt(k) * eps / 10`` for rows of ``k`` values."""
    if a.dtype not in _EPS:
        raise ValueError(f"Invalid dtype: {a.dtype}")
    eps, k = _EPS[a.dtype], a.size(-1)
    largest = max(a.max(), b.max()).item()
    torch.testing.assert_close(a, b, atol=min(1e-2, k * largest * eps * 1e-2), rtol=math.sqrt(k) * eps * 1e-1)
