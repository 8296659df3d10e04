"""The permutation plan without a workspace argument (gmoe_permute_plan_static) gives the bits of
gmoe_permute_plan, through the C ABI, on two calls in a row that share the library's device array
(the second on a smaller input), and refuses sizes beyond its fixed maximum."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _map(T, E, k, seed):
    g = torch.Generator().manual_seed(seed)
    idx = torch.topk(torch.randn(T, E, generator=g), k, dim=1)[1]
    return torch.zeros(T, E, dtype=torch.bool).scatter_(1, idx, True)


def _plan(pkg, dev, rmap, n_out, capacity, static):
    """(dst_map, sorted_indices, row_id_map, counts, offsets) from one of the two entry points."""
    L = pkg._C.lib()
    T, E = rmap.shape
    rmap = rmap.to(dev).contiguous()
    dst = torch.full((T, E), -7, dtype=torch.int32, device=dev)
    si = torch.full((n_out,), -7, dtype=torch.int64, device=dev)
    rid = torch.full((E, T), -7, dtype=torch.int64, device=dev)
    cnt = torch.full((E,), -7, dtype=torch.int64, device=dev)
    off = torch.full((E + 1,), -7, dtype=torch.int64, device=dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    if static:
        rc = L.gmoe_permute_plan_static(rmap.data_ptr(), T, E, capacity, dst.data_ptr(), si.data_ptr(),
                                        n_out, rid.data_ptr(), cnt.data_ptr(), off.data_ptr(), st)
    else:
        ws = torch.empty(max(1, L.gmoe_permute_plan_workspace_bytes(T, E)), dtype=torch.uint8, device=dev)
        rc = L.gmoe_permute_plan(rmap.data_ptr(), T, E, capacity, dst.data_ptr(), si.data_ptr(), n_out,
                                 rid.data_ptr(), cnt.data_ptr(), off.data_ptr(), ws.data_ptr(), st)
    assert rc == 0, rc
    torch.cuda.synchronize(dev)
    return [t.cpu() for t in (dst, si, rid, cnt, off)]


CALLS = [  # two calls in a row on one GPU; the second is smaller and finds the first one's leftovers
    (16384, 8, 2, 0),
    (1000, 64, 8, 0),
    (777, 4, 2, 0),
    (300, 60, 6, 20),   # fixed-capacity blocks (drop and pad)
]


def test_static_plan_matches_workspace_plan(pkg, orc, dev):
    with torch.cuda.device(dev):
        for T, E, k, cap in CALLS:
            print("case", T, E, k, cap, flush=True)
            rmap = _map(T, E, k, seed=T + E)
            n_out = cap * E if cap else T * k
            want = _plan(pkg, dev, rmap, n_out, cap, static=False)
            got = _plan(pkg, dev, rmap, n_out, cap, static=True)
            for w, g in zip(want, got):
                assert torch.equal(w, g)
            if not cap:  # and both agree with the oracle's sorted_indices
                assert torch.equal(got[1], orc.permute(torch.zeros(T, 1), rmap)[1])


def test_static_plan_empty_and_limit(pkg, dev):
    L = pkg._C.lib()
    with torch.cuda.device(dev):
        got = _plan(pkg, dev, torch.zeros(0, 8, dtype=torch.bool), 0, 0, static=True)
        assert got[3].tolist() == [0] * 8 and got[4].tolist() == [0] * 9
        # beyond the fixed maximum: a clear error, nothing launched, outputs untouched
        limit = L.gmoe_permute_plan_static_max_slots()
        E = 512
        T = (limit // E + 1) * 256
        rmap = torch.zeros(T, E, dtype=torch.bool, device=dev)
        dst = torch.full((T, E), -7, dtype=torch.int32, device=dev)
        cnt = torch.full((E,), -7, dtype=torch.int64, device=dev)
        off = torch.full((E + 1,), -7, dtype=torch.int64, device=dev)
        rc = L.gmoe_permute_plan_static(rmap.data_ptr(), T, E, 0, dst.data_ptr(), None, 0, None,
                                        cnt.data_ptr(), off.data_ptr(),
                                        torch.cuda.current_stream(dev).cuda_stream)
        assert rc == -4 and b"maximum" in L.gmoe_status_string(rc)
        torch.cuda.synchronize(dev)
        assert int(cnt[0]) == -7 and int(dst[0, 0]) == -7
        # exactly at the limit it runs
        T = (limit // E) * 256
        rmap = _map(T, E, 2, seed=3)
        want = _plan(pkg, dev, rmap, T * 2, 0, static=False)
        got = _plan(pkg, dev, rmap, T * 2, 0, static=True)
        for w, g in zip(want, got):
            assert torch.equal(w, g)
