"""tqmoe_dispatch_static (the entry point that allocates nothing: its scratch is an array in the library's device image)
against tqmoe_dispatch, through the C ABI, on two calls in a row, the second with a smaller input; then once beyond the
built-in scratch's limit, which must be refused."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tq():
    import tqllm_amd
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    torch.zeros(1, device="cuda")
    err = tqllm_amd.api._err()
    assert tqllm_amd.lib().tqmoe_static_scratch_init(err) == 0, err.message       # the scratch's address, outside any capture
    return tqllm_amd


def both(tq, ids, experts, capacity):
    n, k = ids.shape
    counts, offsets, perm, groups = tq.moe_dispatch(ids, experts, capacity)
    c2 = torch.full_like(counts, -7)
    o2 = torch.full_like(offsets, -7)
    p2 = torch.full_like(perm, -1)
    g2 = torch.full_like(groups, -1) if groups is not None else None
    # device-level free bytes (hipMemGetInfo) around the call: an allocation of any kind inside the library would show, which
    # the caching allocator's own counter would not. The scratch's address has been looked up before (the fixture).
    torch.cuda.synchronize()
    before, before_torch = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    tq.moe_dispatch_into(ids, experts, c2, o2, p2, g2, capacity)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == before and torch.cuda.memory_allocated() == before_torch
    assert torch.equal(c2, counts) and torch.equal(o2, offsets) and torch.equal(p2, perm)
    if groups is not None:
        assert torch.equal(g2, groups)
    return counts


def test_dispatch_static_matches_dispatch_twice_second_smaller(tq):
    rng = np.random.default_rng(77)
    experts = 512
    # first call: 45,056 assignments (44 chunks) with a skewed load; second: 3,000 assignments (3 chunks) of other ids
    p = 1.0 / np.arange(1, experts + 1) ** 1.1
    first = torch.from_numpy(rng.choice(experts, size=(4096, 11), p=p / p.sum()).astype(np.int32)).cuda()
    first[5, 3] = -1                                   # a skipped assignment
    c = both(tq, first, experts, int(4096))
    assert int(c.sum()) == 4096 * 11 - 1
    second = torch.from_numpy(rng.integers(0, experts, size=(300, 10)).astype(np.int32)).cuda()
    both(tq, second, experts, 0)
    third = torch.from_numpy(rng.integers(0, 7, size=(9, 3)).astype(np.int32)).cuda()        # one chunk: no scratch at all
    both(tq, third, 7, 27)
    both(tq, first, experts, 0)                        # and the large one again after the small ones


def test_dispatch_static_two_streams_one_after_the_other(tq):
    """Calls on one GPU share the scratch: issued from two streams they must be ordered by the caller. Ordered with an event,
    the second stream's call (a smaller input) sees none of the first's counts."""
    rng = np.random.default_rng(78)
    experts = 256
    a = torch.from_numpy(rng.integers(0, experts, size=(3000, 8)).astype(np.int32)).cuda()
    b = torch.from_numpy(rng.integers(0, experts, size=(500, 5)).astype(np.int32)).cuda()
    want = [tq.moe_dispatch(t, experts)[:3] for t in (a, b)]
    got = [[torch.full_like(w, -3) for w in ws] for ws in want]
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(s1):
        tq.moe_dispatch_into(a, experts, *got[0])
    done = torch.cuda.Event()
    done.record(s1)
    s2.wait_event(done)
    with torch.cuda.stream(s2):
        tq.moe_dispatch_into(b, experts, *got[1])
    torch.cuda.synchronize()
    for ws, gs in zip(want, got):
        for w, g in zip(ws, gs):
            assert torch.equal(w, g)


def test_dispatch_static_refuses_what_its_scratch_cannot_hold(tq):
    experts = 4096
    n, k = 70000, 4                                    # 274 chunks x 4096 experts > 1,048,576 ints
    ids = torch.zeros((n, k), dtype=torch.int32, device="cuda")
    counts = torch.empty(experts, dtype=torch.int32, device="cuda")
    offsets = torch.empty(experts + 1, dtype=torch.int32, device="cuda")
    perm = torch.empty(n * k, dtype=torch.int32, device="cuda")
    with pytest.raises(tq.TqmoeError) as info:
        tq.moe_dispatch_into(ids, experts, counts, offsets, perm)
    assert info.value.code == -4 and "scratch" in str(info.value)
