"""fp8 (e4m3) inference variant on the GPU (BASELINE config 4).  The reference has
no fp8 path; the oracle is dequantised fp32 math on the same quantised operands,
and the fp32 oracle on the unquantised weights gives the end-to-end accuracy bar:
rel-Frobenius <= 8e-2 (measured 6.5e-2: two e4m3 GEMMs, 3 mantissa bits each, with
per-token and per-channel scales)."""
import pytest
import torch

from oracle import moe_ref
from util import assert_parity, randn, random_group_indices, seeded

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols,dtype", [(7, 128, torch.bfloat16), (300, 4096, torch.bfloat16),
                                             (64, 1000, torch.float32), (33, 14336, torch.float16),
                                             (5, 37, torch.float32)])
def test_quantize_rows_bit_exact(rows, cols, dtype):
    from moe_explore.fp8 import quantize_rows
    x = randn((rows, cols), seeded(rows + cols), dtype, 3.0)
    x[0, :] = 0  # an all-zero row quantises to zeros with the floor scale
    q, s = quantize_rows(x.cuda())
    q_ref, s_ref = moe_ref.quantize_rows_fp8(x)
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


@pytest.mark.parametrize("tiled", [True, False])
@pytest.mark.parametrize("rows,E,K,N,act", [(300, 4, 256, 512, None), (1000, 8, 512, 1024, "swiglu"),
                                            (4096, 8, 1024, 512, "geglu"), (64, 2, 128, 64, "silu"),
                                            (700, 3, 384, 328, None)])
def test_m_grouped_gemm_fp8_plain(rows, E, K, N, act, tiled):
    from moe_explore.fp8 import quantize_rows, quantize_expert_weights, m_grouped_gemm_fp8
    g = seeded(rows + K)
    x = randn((rows, K), g, torch.bfloat16)
    w = randn((E, K, N), g, torch.bfloat16, 0.05)
    gi = random_group_indices(rows, E, g)
    xq, xs = quantize_rows(x.cuda())
    wq = quantize_expert_weights(w.cuda(), tiled=tiled)
    assert wq.tiled == tiled and wq.codes().shape == (E, N, K)
    out = m_grouped_gemm_fp8(xq, xs, wq, gi.cuda(), num_tokens=rows, activation=act)
    # oracle: the same codes, dequantised, fp32 matmul
    xd = xq.cpu().float() * xs.cpu().unsqueeze(1)
    wd = (wq.codes().cpu().float() * wq.scale.cpu().unsqueeze(-1)).transpose(1, 2)
    ref = moe_ref.grouped_matmul_gather_scatter(xd, wd, gi, activation_name=act)
    assert_parity(out, ref, torch.bfloat16, "fp8 gemm vs dequantised oracle", tol=1e-2)
    # the (offline, plain PyTorch) weight quantiser agrees with the oracle's up to the
    # last bit of the fp32 division on the two devices
    q_ref, s_ref = moe_ref.quantize_weight_fp8(w)
    torch.testing.assert_close(wq.scale.cpu(), s_ref, rtol=1e-6, atol=0)
    mismatch = (wq.codes().cpu().view(torch.uint8) != q_ref.view(torch.uint8)).float().mean().item()
    assert mismatch < 1e-2  # a code flips only where x/scale sits on a rounding tie


@pytest.mark.parametrize("tiled", [True, False])
@pytest.mark.parametrize("parts", [2, 4])
def test_m_grouped_gemm_fp8_split_k(parts, tiled):
    """K cut into parts: the stacked partial results add up to the unsplit product (each
    part is rounded to bf16 on its own, so to bf16 accuracy), also through the scatter."""
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.fp8 import quantize_rows, quantize_expert_weights, m_grouped_gemm_fp8
    g = seeded(parts)
    T, E, k, K, N = 150, 4, 2, 1024, 520
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    p = get_token_indices(idx.cuda(), k, E, zero_prefix=True)
    a = randn((T * k, K), g, torch.bfloat16)
    w = randn((E, K, N), g, torch.bfloat16, 0.05)
    aq, as_ = quantize_rows(a.cuda())
    wq = quantize_expert_weights(w.cuda(), tiled=tiled)
    whole = m_grouped_gemm_fp8(aq, as_, wq, p.group_indices, p.indices, scatter=True, num_tokens=T, topk=k)
    split = m_grouped_gemm_fp8(aq, as_, wq, p.group_indices, p.indices, scatter=True, num_tokens=T, topk=k,
                               ksplit=parts)
    assert split.shape == (parts * T * k, N)
    summed = split.float().view(parts, T * k, N).sum(0)
    assert_parity(summed, whole.float().cpu(), torch.bfloat16, "fp8 split K", tol=1e-2)
    # with an activation the split is refused and one part comes back
    one = m_grouped_gemm_fp8(aq, as_, wq, p.group_indices, p.indices, scatter=True, num_tokens=T, topk=k,
                             activation="silu", ksplit=parts)
    assert one.shape == (T * k, N)


@pytest.mark.parametrize("T", [128, 1024])
@pytest.mark.parametrize("act", ["swiglu", "geglu"])
def test_fp8_layer_against_bf16(T, act):
    """Config 4 at reduced d_ff (so that the CPU oracle finishes in seconds): fp8 layer vs
    the fp32 oracle on the unquantised bf16 weights, rel-Frobenius <= 8e-2."""
    from moe_explore.fp8 import Fp8MLPParams, quantize_expert_weights, routed_experts_fp8
    g = seeded(T)
    d, ff, E, k = 4096, 1792, 8, 2
    x = randn((T, d), g, torch.bfloat16)
    w1 = randn((E, d, 2 * ff), g, torch.bfloat16, 0.02)
    w2 = randn((E, ff, d), g, torch.bfloat16, 0.02)
    scores, idx = moe_ref.route_from_logits(torch.randn((T, E), generator=g), k, True, True, torch.bfloat16)
    params = Fp8MLPParams(quantize_expert_weights(w1.cuda()), quantize_expert_weights(w2.cuda()), act)
    out = routed_experts_fp8(x.cuda(), params, scores.cuda(), idx.cuda(), E, k)
    sel = torch.arange(0, T, max(T // 128, 1))
    ref = moe_ref.experts_forward(x[sel], w1, w2, scores[sel], idx[sel], E, k, act)
    err = moe_ref.rel_fro(out[sel.cuda()], ref)
    assert torch.isfinite(out.float()).all()
    assert err <= 8e-2, f"fp8 layer vs bf16-weight oracle: rel-Frobenius {err:.3e}"


def test_fp8_full_size_t8192_runs_and_is_linear_in_scores():
    """Config 4, T=8192 at full width: finite, and halving the routing weights halves
    the output exactly (power-of-two scaling commutes with every rounding)."""
    from moe_explore.fp8 import Fp8MLPParams, quantize_expert_weights, routed_experts_fp8
    dev = "cuda"
    gd = torch.Generator(device=dev); gd.manual_seed(0)
    T, d, ff, E, k = 8192, 4096, 14336, 8, 2
    x = torch.randn((T, d), device=dev, generator=gd).to(torch.bfloat16)
    w1 = torch.empty((E, d, 2 * ff), device=dev, dtype=torch.bfloat16).normal_(0, 0.02, generator=gd)
    w2 = torch.empty((E, ff, d), device=dev, dtype=torch.bfloat16).normal_(0, 0.02, generator=gd)
    scores, idx = moe_ref.route_from_logits(torch.randn((T, E), device=dev, generator=gd), k, True, True,
                                            torch.bfloat16)
    params = Fp8MLPParams(quantize_expert_weights(w1), quantize_expert_weights(w2), "swiglu")
    del w1, w2
    out = routed_experts_fp8(x, params, scores, idx, E, k)
    half = routed_experts_fp8(x, params, scores * 0.5, idx, E, k)
    assert torch.isfinite(out.float()).all()
    assert torch.equal(half.float() * 2, out.float())


@pytest.fixture(scope="module")
def config4_weights():
    """Config-4 weights at full width (d=4096, ff=14336, E=8): N(0, 0.02) bf16 made on the GPU,
    their fp8 quantisation, and an fp32 copy on the host for the oracle."""
    dev = "cuda"
    gd = torch.Generator(device=dev).manual_seed(4)
    d, ff, E = 4096, 14336, 8
    w1 = torch.empty((E, d, 2 * ff), device=dev, dtype=torch.bfloat16).normal_(0, 0.02, generator=gd)
    w2 = torch.empty((E, ff, d), device=dev, dtype=torch.bfloat16).normal_(0, 0.02, generator=gd)
    from moe_explore.fp8 import quantize_expert_weights
    q1, q2 = quantize_expert_weights(w1), quantize_expert_weights(w2)
    host = (w1.cpu().float(), w2.cpu().float())
    del w1, w2
    torch.cuda.empty_cache()
    yield q1, q2, host
    del q1, q2, host
    torch.cuda.empty_cache()


@pytest.mark.parametrize("T,checked", [(128, 32), (1024, 48), (8192, 32)])
@pytest.mark.parametrize("act", ["swiglu", "geglu"])
def test_fp8_layer_full_width_against_bf16_weights(config4_weights, T, checked, act):
    """Config 4 at its real width: T = 128 and 1024 (the weight-streaming regime: split-K down
    projection, tile-major weights) and T = 8192 (256-row tiles, bound by the matrix cores): the
    fp8 layer against the fp32 oracle on the unquantised weights for a subset of tokens (a
    token's output depends on its own row), <= 8e-2."""
    from moe_explore.fp8 import Fp8MLPParams, routed_experts_fp8
    q1, q2, (w1, w2) = config4_weights
    g = seeded(T + len(act))
    d, E, k = 4096, 8, 2
    x = randn((T, d), g, torch.bfloat16)
    scores, idx = moe_ref.route_from_logits(torch.randn((T, E), generator=g), k, True, True, torch.bfloat16)
    out = routed_experts_fp8(x.cuda(), Fp8MLPParams(q1, q2, act), scores.cuda(), idx.cuda(), E, k)
    assert torch.isfinite(out.float()).all()
    sel = torch.randperm(T, generator=g)[:checked]
    ref = moe_ref.experts_forward(x[sel], w1, w2, scores[sel], idx[sel], E, k, act)
    err = moe_ref.rel_fro(out[sel.cuda()], ref)
    assert err <= 8e-2, f"fp8 layer, T={T}, {act}: rel-Frobenius {err:.3e} vs the bf16-weight oracle"


@pytest.mark.parametrize("T", [128, 1024, 8192])
def test_fp8_gate_up_gemm_full_width_against_dequantised_oracle(config4_weights, T):
    """The gate/up fp8 GEMM alone at full width (N = 28672, tile-major weights) against fp32
    products of the SAME codes and scales: rows of two experts, every column."""
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.fp8 import m_grouped_gemm_fp8, quantize_rows
    q1, _, _ = config4_weights
    g = seeded(T)
    d, E, k = 4096, 8, 2
    x = randn((T, d), g, torch.bfloat16)
    _, idx = moe_ref.route_from_logits(torch.randn((T, E), generator=g), k, True, True, torch.bfloat16)
    p = get_token_indices(idx.cuda(), k, E, zero_prefix=True)
    xq, xs = quantize_rows(x.cuda())
    h = m_grouped_gemm_fp8(xq, xs, q1, p.group_indices, p.indices, gather=True, num_tokens=T, topk=k)
    gi, ind = p.group_indices.cpu(), p.indices.cpu()
    xd = xq.cpu().float() * xs.cpu().unsqueeze(1)
    for e in (0, E - 1):
        lo, hi = int(gi[e]), int(gi[e + 1])
        if hi <= lo:
            continue
        # 24 positions spread over the expert's segment (every row block of it at T = 8192)
        rows = torch.unique(torch.linspace(lo, hi - 1, 24).long())
        codes = q1.codes()[e]                                        # [N, K] on the GPU
        wd = (codes.float() * q1.scale[e].unsqueeze(-1)).t().cpu()   # [K, N]
        ref = xd[ind[rows] // k] @ wd
        assert_parity(h[rows.cuda()], ref, torch.bfloat16, f"fp8 gate/up GEMM, expert {e}", tol=1e-2)


@pytest.mark.parametrize("tiled", [True, False])
def test_fp8_many_tiles_odd_column_tile_count_one_k_step(tiled):
    """More than 2048 tiles, so a work item takes two adjacent column tiles, with 65 column
    tiles (the last work item of a row block has one) and K = 128 (one K step a tile: the
    copies of a work item's second tile start before its first step is multiplied); through
    the gather and the scatter."""
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.fp8 import quantize_rows, quantize_expert_weights, m_grouped_gemm_fp8
    g = seeded(65)
    T, E, k, K, N = 4096, 8, 2, 128, 65 * 256
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    p = get_token_indices(idx.cuda(), k, E, zero_prefix=True)
    x = randn((T, K), g, torch.bfloat16)
    w = randn((E, K, N), g, torch.bfloat16, 0.05)
    xq, xs = quantize_rows(x.cuda())
    wq = quantize_expert_weights(w.cuda(), tiled=tiled)
    xd = xq.cpu().float() * xs.cpu().unsqueeze(1)
    wd = (wq.codes().cpu().float() * wq.scale.cpu().unsqueeze(-1)).transpose(1, 2)
    perm, gi = p.indices.cpu(), p.group_indices.cpu()
    out = m_grouped_gemm_fp8(xq, xs, wq, p.group_indices, p.indices, gather=True, num_tokens=T, topk=k)
    ref = moe_ref.grouped_matmul_gather_scatter(xd, wd, gi, perm, gather=True, topk=k)
    assert_parity(out, ref, torch.bfloat16, "fp8 gemm, gathered, 65 column tiles", tol=1e-2)
    rows = out  # [T*k, N] in sorted order: feed them back through the scatter with a narrow weight
    w2 = randn((E, N, 128), g, torch.bfloat16, 0.05)
    aq, as_ = quantize_rows(rows)
    w2q = quantize_expert_weights(w2.cuda(), tiled=tiled)
    out2 = m_grouped_gemm_fp8(aq, as_, w2q, p.group_indices, p.indices, scatter=True, num_tokens=T, topk=k)
    ad = aq.cpu().float() * as_.cpu().unsqueeze(1)
    w2d = (w2q.codes().cpu().float() * w2q.scale.cpu().unsqueeze(-1)).transpose(1, 2)
    ref2 = moe_ref.grouped_matmul_gather_scatter(ad, w2d, gi, perm, scatter=True, topk=k)
    assert_parity(out2, ref2, torch.bfloat16, "fp8 gemm, scattered, K = 65 * 256", tol=1e-2)


def test_fp8_operands_beyond_32_bit_offsets_are_refused():
    """The copy sources are 32-bit offsets from the token matrix (when gathered) and from one
    expert's weights: larger operands are refused before anything is launched (the sizes
    below are only claimed, the buffers are small and never touched)."""
    from moe_explore import _C
    dev = "cuda"
    buf = torch.zeros(4096, device=dev, dtype=torch.uint8)
    scale = torch.ones(1024, device=dev, dtype=torch.float32)
    gi = torch.zeros(3, device=dev, dtype=torch.int32)
    idx = torch.zeros(16, device=dev, dtype=torch.int32)
    lib = _C.load()

    def call(a_rows, K, N, flags):
        return lib.moe_m_grouped_gemm_fp8(
            buf.data_ptr(), scale.data_ptr(), a_rows, K, buf.data_ptr(), scale.data_ptr(), buf.data_ptr(),
            16, N, gi.data_ptr(), idx.data_ptr(), 4, 0, 2, K, N, 1, flags, 0, _C.dtype_code(torch.bfloat16),
            1, 0, _C.stream_of(buf))
    # gathered token matrix of 2^20 rows x 4096 bytes = 4 GiB
    assert call(1 << 20, 4096, 256, _C.GEMM_GATHER_A) == -2  # MOE_ERR_UNSUPPORTED
    # one expert's weights: 2^16 x 2^16 bytes
    assert call(16, 1 << 16, 1 << 16, 0) == -2  # MOE_ERR_UNSUPPORTED
    # within reach: group_indices are all zero, so nothing is computed
    assert call(16, 128, 256, 0) == 0
    torch.cuda.synchronize()
