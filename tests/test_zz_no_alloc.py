"""moe_route_preprocess_noalloc (the entry point that allocates nothing: its per-chunk counts
live in a buffer inside the library) against moe_route_preprocess with a caller workspace,
through the C ABI, bit for bit, on two calls in a row of which the second is smaller (the
buffer then still holds the first call's counts), and against the C oracle."""
import pytest
import torch

from oracle import moe_ref

pytestmark = pytest.mark.gpu


def _both(lib, ids, E):
    """(indices, group_indices, inclusive) of the workspace entry point and of the
    allocation-free one for the same ids."""
    from moe_explore import _C
    R = ids.numel()
    dev = ids.device
    outs = []
    for noalloc in (False, True):
        ind = torch.full((R,), -1, dtype=torch.int64, device=dev)
        gi = torch.full((E + 1,), -1, dtype=torch.int32, device=dev)
        inc = torch.full((E,), -1, dtype=torch.int64, device=dev)
        stream = _C.stream_of(ids)
        if noalloc:
            st = lib.moe_route_preprocess_noalloc(ids.data_ptr(), _C.idx_bytes(ids), R, E, ind.data_ptr(),
                                                  gi.data_ptr(), inc.data_ptr(), stream)
        else:
            nbytes = lib.moe_route_workspace_bytes(R, E)
            ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
            st = lib.moe_route_preprocess(ids.data_ptr(), _C.idx_bytes(ids), R, E, ind.data_ptr(),
                                          gi.data_ptr(), inc.data_ptr(), ws.data_ptr(), ws.numel(), stream)
        _C.check(st, "routing preprocessing")
        outs.append((ind, gi, inc))
    return outs


@pytest.mark.parametrize("first,second", [
    ((98304, 64, torch.int64), (8192, 8, torch.int64)),       # config 3 then config 1
    ((65536, 64, torch.int32), (1000, 64, torch.int32)),      # same E, fewer slots
    ((5000, 160, torch.int64), (4999, 3, torch.int32)),
    ((513, 8, torch.int64), (0, 8, torch.int64)),             # then an empty call
])
def test_noalloc_routing_matches_the_workspace_entry_point(first, second):
    from moe_explore import _C
    lib = _C.load()
    assert lib.moe_route_noalloc_max_bytes() == 4 << 20
    g = torch.Generator().manual_seed(first[0] + second[0])
    for R, E, dtype in (first, second):
        print(f"[noalloc] R={R} E={E} {dtype}", flush=True)
        ids = torch.randint(0, E, (R,), generator=g).to(dtype)
        if R > 100:
            ids[R // 3: R // 3 + 40] = E - 1           # a run of one expert, and
            ids[ids == 1] = 0                          # an expert without slots (E > 1)
        (ind_w, gi_w, inc_w), (ind_n, gi_n, inc_n) = _both(lib, ids.cuda(), E)
        torch.cuda.synchronize()
        assert torch.equal(ind_n, ind_w) and torch.equal(gi_n, gi_w) and torch.equal(inc_n, inc_w)
        gi_ref, ind_ref = moe_ref.get_token_indices(ids, 1, E, zero_prefix=True)
        assert torch.equal(gi_n.cpu(), gi_ref) and torch.equal(ind_n.cpu(), ind_ref)


def test_noalloc_routing_python_wrapper_and_size_limit():
    from moe_explore import _C
    from moe_explore.expert_permute import get_token_indices, get_token_indices_into
    g = torch.Generator().manual_seed(5)
    T, k, E = 3000, 6, 64
    idx = torch.randint(0, E, (T, k), generator=g).cuda()
    want = get_token_indices(idx, k, E, zero_prefix=True)
    ind = torch.empty(T * k, dtype=torch.int64, device="cuda")
    gi = torch.empty(E + 1, dtype=torch.int32, device="cuda")
    got = get_token_indices_into(idx, E, ind, gi)
    assert torch.equal(got.indices, want.indices) and torch.equal(got.group_indices, want.group_indices)
    # beyond the resident buffer: ceil(R / 512) * E words > 2**20 -> a clear error, nothing launched
    lib = _C.load()
    R, E_big = 512 * 1024, 2048
    assert lib.moe_route_workspace_bytes(R, E_big) > lib.moe_route_noalloc_max_bytes()
    st = lib.moe_route_preprocess_noalloc(idx.data_ptr(), 8, R, E_big, ind.data_ptr(), gi.data_ptr(), None,
                                          _C.stream_of(idx))
    assert st == -3 and b"scratch" in lib.moe_last_error_string()
    with pytest.raises(_C.MoeHipError):
        big = torch.zeros(R, dtype=torch.int64, device="cuda")
        get_token_indices_into(big, E_big, torch.empty(R, dtype=torch.int64, device="cuda"),
                               torch.empty(E_big + 1, dtype=torch.int32, device="cuda"))


def test_noalloc_routing_captured_into_a_graph_and_replayed():
    """The call recorded into a HIP graph (after one eager call, which looks up the resident
    buffer) and replayed twice in sequence on one stream with new expert ids each time, with
    eager work of the same entry point between the replays: every replay equals the workspace
    entry point on the ids of that moment."""
    from moe_explore.expert_permute import get_token_indices, get_token_indices_into
    g = torch.Generator().manual_seed(11)
    T, k, E = 2000, 4, 32
    ids = torch.randint(0, E, (T, k), generator=g).cuda()
    ind = torch.empty(T * k, dtype=torch.int64, device="cuda")
    gi = torch.empty(E + 1, dtype=torch.int32, device="cuda")
    get_token_indices_into(ids, E, ind, gi)              # eager: resolves the buffer's address
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        get_token_indices_into(ids, E, ind, gi)
    small = torch.randint(0, 5, (300,), generator=g).cuda()
    for step in range(3):
        ids.copy_(torch.randint(0, E, (T, k), generator=g))
        ind.fill_(-1)
        gi.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        want = get_token_indices(ids, k, E, zero_prefix=True)
        assert torch.equal(ind, want.indices) and torch.equal(gi, want.group_indices), f"replay {step}"
        # eager use of the same buffer between the replays (other sizes: other counts in it)
        e_ind = torch.empty(300, dtype=torch.int64, device="cuda")
        e_gi = torch.empty(6, dtype=torch.int32, device="cuda")
        get_token_indices_into(small, 5, e_ind, e_gi)
        torch.cuda.synchronize()
        e_want = get_token_indices(small, 1, 5, zero_prefix=True)
        assert torch.equal(e_ind, e_want.indices) and torch.equal(e_gi, e_want.group_indices)


def test_noalloc_routing_from_two_streams_back_to_back():
    """Calls issued on two streams without any synchronisation between them share the one
    resident buffer; the entry point orders them itself (the second stream waits for the first
    call's launches), so both results are right."""
    from moe_explore.expert_permute import get_token_indices, get_token_indices_into
    g = torch.Generator().manual_seed(23)
    cases = [(98304, 64), (60000, 48), (98304, 64), (30000, 8)]
    ids = [torch.randint(0, E, (R,), generator=g).cuda() for R, E in cases]
    outs = [(torch.full((R,), -1, dtype=torch.int64, device="cuda"),
             torch.full((E + 1,), -1, dtype=torch.int32, device="cuda")) for R, E in cases]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for rep in range(3):
        for i, ((R, E), x, (ind, gi)) in enumerate(zip(cases, ids, outs)):
            with torch.cuda.stream(streams[i % 2]):
                get_token_indices_into(x, E, ind, gi)
    torch.cuda.synchronize()
    for (R, E), x, (ind, gi) in zip(cases, ids, outs):
        want = get_token_indices(x, 1, E, zero_prefix=True)
        assert torch.equal(ind, want.indices) and torch.equal(gi, want.group_indices)
