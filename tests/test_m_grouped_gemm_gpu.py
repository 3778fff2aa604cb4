"""M-grouped GEMM on the GPU against the fp32-accumulating oracle.
Cases follow the reference's tests/test_m_grouped_gemm.py:12-26, 66-72 (plain,
gather, scatter + combine) and add fp16 / fp32, ragged and empty groups, a
single expert, odd shapes, the fused combine and the transposed-weight product."""
import math

import pytest
import torch

from oracle import moe_ref
from util import assert_parity, randn, random_group_indices, seeded

pytestmark = pytest.mark.gpu

PLAIN_CASES = [
    (10, 4, 128, 128, None, torch.bfloat16),
    (200, 4, 512, 512, None, torch.bfloat16),
    (200, 4, 512, 512, "gelu", torch.bfloat16),
    (200, 4, 512, 512, "silu", torch.bfloat16),
    (200, 4, 512, 512, "swiglu", torch.bfloat16),
    (200, 4, 512, 512, "geglu", torch.bfloat16),
    (1000, 16, 1024, 1024, "gelu", torch.bfloat16),
    (1000, 16, 1024, 1024, "swiglu", torch.bfloat16),
    (16000, 16, 1024, 1024, "geglu", torch.bfloat16),
    (1000, 1, 1024, 1024, "geglu", torch.bfloat16),   # single expert (broken in the reference)
    (1000, 2, 300, 20, "gelu", torch.bfloat16),       # odd sizes -> scalar-FMA kernel
    (1000, 2, 304, 24, "approx_gelu", torch.bfloat16),
    (700, 5, 264, 520, "swiglu", torch.float16),      # K, N multiples of 8 but not of the tile
    (300, 3, 256, 384, None, torch.float16),
    (513, 8, 256, 512, "swiglu", torch.float32),
    (100, 4, 100, 36, "geglu", torch.float32),
    (4096, 8, 512, 1024, None, torch.bfloat16),       # large groups -> 256-row tiles
]


def _params(weight, gi, perm, gather, scatter, num_tokens, topk, scales=None, activation=None):
    from moe_explore.triton_kernels.m_grouped_gemm import MGroupedGEMMParams
    return MGroupedGEMMParams(weight, gi, perm, gather, scatter, num_tokens, topk, scales=scales,
                              activation=activation)


@pytest.mark.parametrize("num_tokens,num_experts,K,N,activation,dtype", PLAIN_CASES)
def test_m_grouped_gemm(num_tokens, num_experts, K, N, activation, dtype):
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(num_tokens * 7 + K)
    x = randn((num_tokens, K), g, dtype)
    w = randn((num_experts, K, N), g, dtype, 1.0 / math.sqrt(N))
    gi = random_group_indices(num_tokens, num_experts, g)
    out = m_grouped_gemm(x.cuda(), _params(w.cuda(), gi.cuda(), None, False, False, num_tokens, 1,
                                           activation=activation))
    ref = moe_ref.grouped_matmul_gather_scatter(x, w, gi, activation_name=activation)
    assert out.shape == ref.shape and out.dtype == dtype
    assert_parity(out, ref, dtype, "m_grouped_gemm")


def test_all_ones_known_answer():
    """128^3 all-ones problems give 128 everywhere (reference csrc/cutlass_group_gemm.cu:211-212)."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    E = 10
    x = torch.ones((E * 128, 128), dtype=torch.float16, device="cuda")
    w = torch.ones((E, 128, 128), dtype=torch.float16, device="cuda")
    gi = (torch.arange(E + 1, dtype=torch.int32) * 128).cuda()
    out = m_grouped_gemm(x, _params(w, gi, None, False, False, E * 128, 1))
    assert torch.equal(out, torch.full_like(out, 128.0))


def test_perfect_routing_equals_bmm():
    """Equal groups reduce to a batched matmul (reference bench_m_grouped_gemm.py:211-223)."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    E, m, K, N = 8, 256, 512, 768
    g = seeded(9)
    x = randn((E * m, K), g, torch.bfloat16).cuda()
    w = randn((E, K, N), g, torch.bfloat16, 0.05).cuda()
    gi = (torch.arange(E + 1, dtype=torch.int32) * m).cuda()
    out = m_grouped_gemm(x, _params(w, gi, None, False, False, E * m, 1))
    ref = torch.bmm(x.view(E, m, K).float(), w.float()).view(E * m, N)
    assert_parity(out, ref, torch.bfloat16, "bmm")


ROUTED_CASES = [
    (10, 4, 2, 128, 128, None, torch.bfloat16),
    (200, 4, 2, 512, 512, None, torch.bfloat16),
    (200, 4, 2, 512, 512, "gelu", torch.bfloat16),
    (200, 4, 2, 512, 512, "swiglu", torch.bfloat16),
    (200, 4, 2, 512, 512, "geglu", torch.bfloat16),
    (999, 64, 8, 256, 512, "swiglu", torch.float16),
    (300, 8, 2, 200, 100, "geglu", torch.float32),
    (2048, 8, 2, 512, 1024, "swiglu", torch.bfloat16),
]


def _routing(num_tokens, num_experts, topk, g, dtype):
    logits = torch.randn((num_tokens, num_experts), generator=g)
    scores, idx = torch.topk(torch.softmax(logits, -1), topk, dim=-1, sorted=False)
    return scores.to(dtype), idx


@pytest.mark.parametrize("num_tokens,num_experts,topk,K,N,activation,dtype", ROUTED_CASES)
def test_m_grouped_gemm_gather(num_tokens, num_experts, topk, K, N, activation, dtype):
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(num_tokens + K + 1)
    x = randn((num_tokens, K), g, dtype)
    w = randn((num_experts, K, N), g, dtype, 1.0 / math.sqrt(N))
    _, idx = _routing(num_tokens, num_experts, topk, g, dtype)
    p = get_token_indices(idx.view(-1).cuda(), topk, num_experts, zero_prefix=True)
    out, pre = m_grouped_gemm(
        x.cuda(), _params(w.cuda(), p.group_indices, p.indices, True, False, num_tokens, topk,
                          activation=activation), save_preact=True)
    ref, ref_pre = moe_ref.grouped_matmul_gather_scatter(
        x, w, p.group_indices, p.indices, gather=True, num_tokens=num_tokens, topk=topk,
        activation_name=activation, return_preact=True)
    assert_parity(out, ref, dtype, "gather")
    assert_parity(pre, ref_pre, dtype, "gather pre-activation")


@pytest.mark.parametrize("num_tokens,num_experts,topk,K,N,activation,dtype", ROUTED_CASES)
@pytest.mark.parametrize("fused", [False, True])
def test_m_grouped_gemm_scatter(num_tokens, num_experts, topk, K, N, activation, dtype, fused):
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.functional.scale_and_reduce import scale_and_reduce
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(num_tokens + K + 2)
    R = num_tokens * topk
    x = randn((R, K), g, dtype)
    w = randn((num_experts, K, N), g, dtype, 1.0 / math.sqrt(N))
    scores, idx = _routing(num_tokens, num_experts, topk, g, dtype)
    p = get_token_indices(idx.view(-1).cuda(), topk, num_experts, zero_prefix=True)
    params = _params(w.cuda(), p.group_indices, p.indices, False, True, num_tokens, topk,
                     scales=scores.cuda(), activation=activation)
    if fused:
        out = m_grouped_gemm(x.cuda(), params, combine=True)
    else:
        out = m_grouped_gemm(x.cuda(), params)
        assert out.shape[0] == R
        out = scale_and_reduce(out, params.scales, num_tokens, topk, out.size(-1))
    ref = moe_ref.grouped_matmul_gather_scatter(
        x, w, p.group_indices, p.indices, scatter=True, num_tokens=num_tokens, topk=topk,
        scales=scores, activation_name=activation)
    assert out.shape == ref.shape and out.dtype == dtype
    assert_parity(out, ref, dtype, "scatter+combine")


@pytest.mark.parametrize("dtype,K,N", [(torch.bfloat16, 512, 256), (torch.float16, 264, 520),
                                       (torch.float32, 96, 40)])
def test_transposed_weight(dtype, K, N):
    """a @ w[e]^T with w stored [E, N, K] (the dX products of the backward pass)."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(K + N)
    rows, E = 777, 6
    x = randn((rows, K), g, dtype)
    w = randn((E, N, K), g, dtype, 0.05)
    gi = random_group_indices(rows, E, g)
    out = m_grouped_gemm(x.cuda(), _params(w.cuda(), gi.cuda(), None, False, False, rows, 1),
                         transpose_weight=True)
    ref = moe_ref.grouped_matmul_gather_scatter(x, w.transpose(1, 2), gi)
    assert_parity(out, ref, dtype, "transposed weight")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("activation", [None, "silu", "gelu", "approx_gelu", "swiglu", "geglu"])
@pytest.mark.parametrize("transposed", [False, True])
def test_large_ragged_groups_every_epilogue(dtype, activation, transposed):
    """Groups of 512+ rows on average take the 256-row tiles on 16x16x32 MFMAs: every
    epilogue and both weight layouts, with an empty group, a 5-row group, a group that ends
    one row into a tile and one that ends 17 rows into a 16-row block."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    K, N = 320, 512
    sizes = [1025, 0, 5, 785, 1000, 529]
    rows, E = sum(sizes), len(sizes)
    g = seeded(rows + (7 if transposed else 0))
    gi = torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32)
    x = randn((rows, K), g, dtype)
    if transposed:
        w = randn((E, N, K), g, dtype, 0.05)
        wv, wref = w.cuda(), w.transpose(1, 2)
    else:
        w = randn((E, K, N), g, dtype, 0.05)
        wv, wref = w.cuda(), w
    out = m_grouped_gemm(x.cuda(), _params(wv, gi.cuda(), None, False, False, rows, 1,
                                           activation=activation), transpose_weight=transposed)
    ref = moe_ref.grouped_matmul_gather_scatter(x, wref, gi, activation_name=activation)
    assert out.shape == ref.shape
    assert_parity(out.cpu(), ref, dtype, f"{activation} transposed={transposed}")


@pytest.mark.parametrize("sizes", [[1025, 0, 5, 785, 1000, 529], [130, 0, 3, 64, 257, 31]])
@pytest.mark.parametrize("K,N", [(28, 36), (36, 520), (100, 264), (256, 512)])
@pytest.mark.parametrize("activation", [None, "silu", "gelu", "approx_gelu", "swiglu", "geglu"])
@pytest.mark.parametrize("transposed", [False, True])
def test_fp32_matrix_core_kernel(sizes, K, N, activation, transposed):
    """fp32 with K, N multiples of 4 runs on 32x32x2 fp32 MFMAs: both tile heights (rows an
    expert above and below 256), both weight layouts, every epilogue, K of one partial step,
    a step and a partial one, several steps with a tail and whole steps, column tiles that are
    partly outside the matrix; empty, tiny and tile-straddling groups."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    dtype = torch.float32
    rows, E = sum(sizes), len(sizes)
    g = seeded(rows + K * 3 + N + (7 if transposed else 0))
    gi = torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32)
    x = randn((rows, K), g, dtype)
    w = randn((E, N, K) if transposed else (E, K, N), g, dtype, 0.1)
    out = m_grouped_gemm(x.cuda(), _params(w.cuda(), gi.cuda(), None, False, False, rows, 1,
                                           activation=activation), transpose_weight=transposed)
    ref = moe_ref.grouped_matmul_gather_scatter(x, w.transpose(1, 2) if transposed else w, gi,
                                                activation_name=activation)
    assert out.shape == ref.shape
    assert_parity(out.cpu(), ref, dtype, f"fp32 K={K} N={N} {activation} transposed={transposed}")


@pytest.mark.parametrize("num_tokens,num_experts,topk", [(300, 8, 2), (3000, 4, 2)])
@pytest.mark.parametrize("activation", [None, "swiglu"])
def test_fp32_matrix_core_kernel_gather_scatter_combine(num_tokens, num_experts, topk, activation):
    """The fp32 MFMA kernel with the fused row gather and saved pre-activation, the row
    scatter and the weighted scatter-add."""
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.functional.scale_and_reduce import scale_and_reduce
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    dtype, K, N = torch.float32, 200, 104
    g = seeded(num_tokens + 5)
    x = randn((num_tokens, K), g, dtype)
    w = randn((num_experts, K, N), g, dtype, 1.0 / math.sqrt(N))
    scores, idx = _routing(num_tokens, num_experts, topk, g, dtype)
    p = get_token_indices(idx.view(-1).cuda(), topk, num_experts, zero_prefix=True)
    out, pre = m_grouped_gemm(
        x.cuda(), _params(w.cuda(), p.group_indices, p.indices, True, False, num_tokens, topk,
                          activation=activation), save_preact=True)
    ref, ref_pre = moe_ref.grouped_matmul_gather_scatter(
        x, w, p.group_indices, p.indices, gather=True, num_tokens=num_tokens, topk=topk,
        activation_name=activation, return_preact=True)
    assert_parity(out, ref, dtype, "fp32 gather")
    assert_parity(pre, ref_pre, dtype, "fp32 gather pre-activation")

    xs = randn((num_tokens * topk, K), g, dtype)
    params = _params(w.cuda(), p.group_indices, p.indices, False, True, num_tokens, topk,
                     scales=scores.cuda(), activation=activation)
    ref = moe_ref.grouped_matmul_gather_scatter(
        xs, w, p.group_indices, p.indices, scatter=True, num_tokens=num_tokens, topk=topk,
        scales=scores, activation_name=activation)
    fused = m_grouped_gemm(xs.cuda(), params, combine=True)
    assert_parity(fused, ref, dtype, "fp32 scatter-add")
    rows = m_grouped_gemm(xs.cuda(), params)
    two_pass = scale_and_reduce(rows, params.scales, num_tokens, topk, rows.size(-1))
    assert_parity(two_pass, ref, dtype, "fp32 scatter + combine")


@pytest.mark.parametrize("K,N", [(64, 272), (128, 528), (192, 1040)])
@pytest.mark.parametrize("activation", [None, "swiglu"])
@pytest.mark.parametrize("transposed", [False, True])
def test_large_groups_short_k_and_ragged_n(K, N, activation, transposed):
    """The same kernels with one to three K steps (the copy pipeline's start-up and
    wind-down paths) and a last column tile that is only partly inside the matrix."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    dtype = torch.bfloat16
    sizes = [700, 515, 1300, 600]
    rows, E = sum(sizes), len(sizes)
    g = seeded(K * 7 + N)
    gi = torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32)
    x = randn((rows, K), g, dtype)
    w = randn((E, N, K) if transposed else (E, K, N), g, dtype, 0.1)
    out = m_grouped_gemm(x.cuda(), _params(w.cuda(), gi.cuda(), None, False, False, rows, 1,
                                           activation=activation), transpose_weight=transposed)
    ref = moe_ref.grouped_matmul_gather_scatter(x, w.transpose(1, 2) if transposed else w, gi,
                                                activation_name=activation)
    assert_parity(out.cpu(), ref, dtype, f"K={K} N={N} {activation} transposed={transposed}")


def test_fused_combine_is_deterministic_for_top2():
    """Two fp32 atomic adds into a zeroed accumulator commute: bit-identical reruns."""
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(77)
    T, E, k, K, N = 1024, 8, 2, 256, 512
    x = randn((T * k, K), g, torch.bfloat16).cuda()
    w = randn((E, K, N), g, torch.bfloat16, 0.05).cuda()
    scores, idx = _routing(T, E, k, g, torch.bfloat16)
    p = get_token_indices(idx.cuda(), k, E, zero_prefix=True)
    params = _params(w, p.group_indices, p.indices, False, True, T, k, scales=scores.cuda())
    a = m_grouped_gemm(x, params, combine=True)
    b = m_grouped_gemm(x, params, combine=True)
    assert torch.equal(a, b)


def test_argument_errors():
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    x = torch.zeros((4, 8), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((2, 16, 8), dtype=torch.bfloat16, device="cuda")
    gi = torch.tensor([0, 2, 4], dtype=torch.int32, device="cuda")
    with pytest.raises(AssertionError):
        m_grouped_gemm(x, _params(w, gi, None, False, False, 4, 1))       # K mismatch
    with pytest.raises(AssertionError):
        m_grouped_gemm(x[0], _params(w, gi, None, False, False, 4, 1))    # 1-D token
    w2 = torch.zeros((2, 8, 8), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(AssertionError):
        m_grouped_gemm(x, _params(w2, gi, None, True, False, 4, 1))       # gather without indices


@pytest.mark.parametrize("ksplit,K", [(2, 1024), (4, 1024), (2, 320)])
def test_split_k_partials_add_up(ksplit, K):
    """ksplit > 1 stores one partial product per K part; scale_and_reduce adds them.
    K = 320 cannot be cut into whole 64-steps: the wrapper falls back to one part."""
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.functional.scale_and_reduce import scale_and_reduce
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(K + ksplit)
    T, E, k, N = 700, 8, 2, 512
    x = randn((T * k, K), g, torch.bfloat16)
    w = randn((E, K, N), g, torch.bfloat16, 1.0 / math.sqrt(N))
    scores, idx = _routing(T, E, k, g, torch.bfloat16)
    p = get_token_indices(idx.cuda(), k, E, zero_prefix=True)
    params = _params(w.cuda(), p.group_indices, p.indices, False, True, T, k, scales=scores.cuda())
    y = m_grouped_gemm(x.cuda(), params, ksplit=ksplit)
    parts = y.size(0) // (T * k)
    assert parts == (ksplit if K % (64 * ksplit) == 0 else 1)
    out = scale_and_reduce(y, params.scales, T, k, N, nsplit=parts)
    ref = moe_ref.grouped_matmul_gather_scatter(x, w, p.group_indices, p.indices, scatter=True,
                                                num_tokens=T, topk=k, scales=scores)
    assert_parity(out, ref, torch.bfloat16, "split K")


def test_tile_counters_are_clean_after_every_launch():
    """The MFMA kernel's resident workgroups draw their tiles from device-side counters that
    each launch clears when it is done; launches take the counter sets in turn, so a set is
    used again every 1024 launches.  2200 launches go round the ring twice and more: every
    result must be the first one, bit for bit."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(77)
    T, E, K, N = 600, 5, 128, 512
    x = randn((T, K), g, torch.bfloat16).cuda()
    w = randn((E, K, N), g, torch.bfloat16, 1.0 / math.sqrt(N)).cuda()
    gi = random_group_indices(T, E, g).cuda()
    p = _params(w, gi, None, False, False, T, 1, activation="swiglu")
    first = m_grouped_gemm(x, p)
    ref = moe_ref.grouped_matmul_gather_scatter(x.cpu(), w.cpu(), gi.cpu(), activation_name="swiglu")
    assert_parity(first, ref, torch.bfloat16, "first launch")
    out = torch.empty_like(first)
    for i in range(2200):
        out.fill_(float("nan"))
        m_grouped_gemm(x, p, out=out)
        if i % 100 == 99 or i >= 2190:
            assert torch.equal(out, first), f"launch {i + 1} differs from the first"


def test_launches_on_two_streams_do_not_share_tile_counters():
    """Two launches in flight at once (two streams) each have a counter set of their own."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(78)
    T, E, K, N = 6000, 4, 512, 1024
    xs, ps, serial = [], [], []
    for s in range(2):
        x = randn((T, K), g, torch.bfloat16).cuda()
        w = randn((E, K, N), g, torch.bfloat16, 1.0 / math.sqrt(N)).cuda()
        gi = random_group_indices(T, E, g).cuda()
        xs.append(x)
        ps.append(_params(w, gi, None, False, False, T, 1, activation=None))
        serial.append(m_grouped_gemm(x, ps[-1]))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [torch.empty_like(serial[0]), torch.empty_like(serial[1])]
    for rep in range(20):
        for s in range(2):
            with torch.cuda.stream(streams[s]):
                m_grouped_gemm(xs[s], ps[s], out=outs[s])
    torch.cuda.synchronize()
    for s in range(2):
        assert torch.equal(outs[s], serial[s]), f"stream {s}"


def _graph_of(fn, warmups=2):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(warmups):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn()
    return graph, out


def test_captured_launches_own_no_tile_counters():
    """A launch recorded into a HIP graph takes its tile ids in strides of the grid instead of
    from a queue set, so replays share no device state with anything: two graphs of the same
    GEMM replayed on two streams at once, next to eager launches of it on a third and fourth,
    all give the serial result; and a graph captured before 1500 eager launches (more than
    there are queue sets) still replays bit-exactly afterwards."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(79)
    T, E, K, N = 5000, 4, 512, 1024
    x = randn((T, K), g, torch.bfloat16).cuda()
    w = randn((E, K, N), g, torch.bfloat16, 1.0 / math.sqrt(N)).cuda()
    gi = random_group_indices(T, E, g).cuda()
    p = _params(w, gi, None, False, False, T, 1, activation="swiglu")
    with torch.no_grad():
        serial = m_grouped_gemm(x, p).clone()
        graphs = [_graph_of(lambda: m_grouped_gemm(x, p)) for _ in range(2)]
        torch.cuda.synchronize()
        streams = [torch.cuda.Stream() for _ in range(4)]
        eager = [torch.empty_like(serial) for _ in range(2)]
        for rep in range(10):
            for i, (graph, out) in enumerate(graphs):
                with torch.cuda.stream(streams[i]):
                    graph.replay()
            for i in range(2):
                with torch.cuda.stream(streams[2 + i]):
                    m_grouped_gemm(x, p, out=eager[i])
            if rep % 3 == 2:
                torch.cuda.synchronize()
                for i, (_, out) in enumerate(graphs):
                    assert torch.equal(out, serial), f"graph {i}, round {rep}"
                    out.fill_(float("nan"))
                for i in range(2):
                    assert torch.equal(eager[i], serial), f"eager stream {i}, round {rep}"
        torch.cuda.synchronize()
        # many eager launches later the first graph is still good
        scratch = torch.empty_like(serial)
        for _ in range(1500):
            m_grouped_gemm(x, p, out=scratch)
        graph, out = graphs[0]
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, serial) and torch.equal(scratch, serial)


def test_many_streams_each_get_a_queue_set():
    """Eager launches on 24 streams in flight together."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(80)
    T, E, K, N = 3000, 4, 256, 512
    x = randn((T, K), g, torch.bfloat16).cuda()
    w = randn((E, K, N), g, torch.bfloat16, 1.0 / math.sqrt(N)).cuda()
    gi = random_group_indices(T, E, g).cuda()
    p = _params(w, gi, None, False, False, T, 1, activation=None)
    serial = m_grouped_gemm(x, p).clone()
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(24)]
    outs = [torch.empty_like(serial) for _ in streams]
    for rep in range(5):
        for s, o in zip(streams, outs):
            with torch.cuda.stream(s):
                m_grouped_gemm(x, p, out=o)
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        assert torch.equal(o, serial), f"stream {i}"


def test_split_k_with_transposed_weights():
    """ksplit = 2 on the K-contiguous (transposed) weight view, the form the dX GEMM of the
    backward pass runs at K = 2 * d_ff; the two partial products add up to the unsplit one."""
    from moe_explore.functional.scale_and_reduce import scale_and_reduce
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(81)
    T, E, K, N, topk = 1536, 4, 1024, 512, 2
    R = T * topk
    a = randn((R, K), g, torch.bfloat16).cuda()
    w = randn((E, N, K), g, torch.bfloat16, 1.0 / math.sqrt(K)).cuda()      # [E, N, K]: used as w^T
    gi = random_group_indices(R, E, g).cuda()
    perm = torch.randperm(R, generator=g).cuda()
    p = _params(w, gi, perm, False, True, T, topk)
    whole = m_grouped_gemm(a, p, transpose_weight=True)
    parts = m_grouped_gemm(a, p, transpose_weight=True, ksplit=2)
    assert parts.shape == (2 * R, N), "the split was declined"
    ref = moe_ref.grouped_matmul_gather_scatter(a.cpu(), w.transpose(1, 2).cpu(), gi.cpu(), perm.cpu(),
                                                scatter=True, num_tokens=T, topk=topk)
    assert_parity(parts[:R].float() + parts[R:].float(), ref, torch.bfloat16, "sum of the K parts")
    assert_parity(whole, ref, torch.bfloat16, "unsplit")
    summed = scale_and_reduce(parts, None, T, topk, N, nsplit=2)
    want = ref.view(T, topk, N).sum(1)
    assert_parity(summed, want, torch.bfloat16, "scale_and_reduce over parts and top-k")


def _group_indices_of(sizes):
    return torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32)


# rows per expert that exercise every case of the two tile orders: no rows, one short block, a
# last block of 1, 128, 129 and 256 rows behind full ones, exactly four and eight blocks, five
# and nine (a band of four and a remainder)
TILE_ORDER_SIZES = [
    [1036, 0, 5, 1024, 257, 384, 385, 2048, 2049, 1280, 1, 512],
    [300, 260, 130, 0, 0, 769, 1152, 255, 256, 513],
]


@pytest.mark.parametrize("sizes", TILE_ORDER_SIZES)
@pytest.mark.parametrize("transposed", [False, True])
@pytest.mark.parametrize("activation", [None, "swiglu"])
def test_expert_aligned_bands_with_long_k(sizes, transposed, activation):
    """K = 4096 without split K: bands of four row blocks that stay inside one expert (padding
    slots in an expert's last band are skipped).  Every expert on its own against the oracle."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(sum(sizes) + transposed)
    R, E, K, N = sum(sizes), len(sizes), 4096, 512
    x = randn((R, K), g, torch.bfloat16)
    w = randn((E, K, N), g, torch.bfloat16, 1.0 / math.sqrt(K))
    gi = _group_indices_of(sizes)
    wc = w.cuda() if not transposed else w.transpose(1, 2).contiguous().cuda()
    out = m_grouped_gemm(x.cuda(), _params(wc, gi.cuda(), None, False, False, R, 1, activation=activation),
                         transpose_weight=transposed)
    ref = moe_ref.grouped_matmul_gather_scatter(x, w, gi, activation_name=activation)
    assert_parity(out, ref, torch.bfloat16, "bands, all rows")
    for e, n in enumerate(sizes):
        if n:
            lo = int(gi[e])
            assert_parity(out[lo:lo + n], ref[lo:lo + n], torch.bfloat16, f"expert {e} ({n} rows)")
            last = lo + (n - 1) // 256 * 256     # the expert's last row block on its own
            assert_parity(out[last:lo + n], ref[last:lo + n], torch.bfloat16, f"last block of expert {e}")


@pytest.mark.parametrize("sizes", TILE_ORDER_SIZES)
@pytest.mark.parametrize("transposed", [False, True])
def test_even_last_row_blocks_with_split_k(sizes, transposed):
    """Split K: a group whose last row block would hold at most 128 rows cuts its last two
    blocks evenly instead; every row is still computed exactly once in each K part."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(sum(sizes) + 7 + transposed)
    R, E, K, N = sum(sizes), len(sizes), 4096, 256
    x = randn((R, K), g, torch.bfloat16)
    w = randn((E, K, N), g, torch.bfloat16, 1.0 / math.sqrt(K))
    gi = _group_indices_of(sizes)
    perm = torch.randperm(R, generator=g)
    wc = w.cuda() if not transposed else w.transpose(1, 2).contiguous().cuda()
    p = _params(wc, gi.cuda(), perm.cuda(), False, True, R, 1)
    parts = m_grouped_gemm(x.cuda(), p, transpose_weight=transposed, ksplit=2)
    assert parts.shape == (2 * R, N), "the split was declined"
    ref = moe_ref.grouped_matmul_gather_scatter(x, w, gi, perm, scatter=True, num_tokens=R, topk=1)
    halves = [moe_ref.grouped_matmul_gather_scatter(x[:, h * 2048:(h + 1) * 2048], w[:, h * 2048:(h + 1) * 2048],
                                                    gi, perm, scatter=True, num_tokens=R, topk=1)
              for h in (0, 1)]
    assert_parity(parts[:R], halves[0], torch.bfloat16, "first K part")
    assert_parity(parts[R:], halves[1], torch.bfloat16, "second K part")
    total = parts[:R].float() + parts[R:].float()
    assert_parity(total, ref, torch.bfloat16, "sum of the K parts")
    for e, n in enumerate(sizes):
        if n:
            rows = perm[int(gi[e]):int(gi[e]) + n]
            assert_parity(total[rows.cuda()], ref[rows], torch.bfloat16, f"expert {e} ({n} rows)")


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("ksplit", [1, 2])
def test_tile_orders_with_many_random_groups(seed, ksplit):
    """More experts than one pass of the tile lookup scans (64), random group sizes from 0 to a
    few row blocks, K = 4096: expert-aligned bands (ksplit 1) and the even last pair of row
    blocks (ksplit 2) must visit every row block exactly once."""
    from moe_explore.triton_kernels.m_grouped_gemm import m_grouped_gemm
    g = seeded(100 + seed)
    E, K, N = 150, 4096, 256
    sizes = torch.randint(0, 700, (E,), generator=g)
    sizes[torch.randint(0, E, (20,), generator=g)] = 0
    sizes[torch.randint(0, E, (5,), generator=g)] = torch.tensor([256, 512, 1024, 1, 1300])
    sizes = sizes.tolist()
    R = sum(sizes)
    x = randn((R, K), g, torch.bfloat16)
    w = randn((E, K, N), g, torch.bfloat16, 1.0 / math.sqrt(K))
    gi = _group_indices_of(sizes)
    out = m_grouped_gemm(x.cuda(), _params(w.cuda(), gi.cuda(), None, False, False, R, 1), ksplit=ksplit)
    if ksplit == 2:
        assert out.shape == (2 * R, N)
        out = out[:R].float() + out[R:].float()
    ref = moe_ref.grouped_matmul_gather_scatter(x, w, gi)
    assert_parity(out, ref, torch.bfloat16, "all rows")
    # row by row: a row block visited twice or not at all shows as a row that is off
    err = (out.float().cpu() - ref).norm(dim=1) / ref.norm(dim=1).clamp_min(1e-6)
    assert err.max().item() <= 2e-2, f"row {int(err.argmax())} is off by {err.max().item():.3e}"
