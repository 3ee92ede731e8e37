"""apt_relabel_static (scratch in a fixed device array of the library, nothing allocated) against
apt_relabel on the same inputs, through the C ABI: two calls in a row, the second smaller, so that
whatever the first call left in the shared array must not leak into the second."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(rng, ns, nn, id_range, pad=0.1):
    seeds = rng.integers(0, id_range, size=ns).astype(np.int64)
    nbr = rng.integers(0, id_range, size=nn).astype(np.int64)
    nbr[rng.random(nn) < pad] = -1
    return torch.from_numpy(seeds).to(DEV), torch.from_numpy(nbr).to(DEV)


def _static(capi, seeds, nbr, ns_dev=None, stride=0):
    L = capi.lib()
    ns, nn = seeds.numel(), nbr.numel()
    uniq = torch.full((ns + nn,), -7, dtype=torch.int64, device=DEV)
    rel = torch.full((nn,), -7, dtype=torch.int64, device=DEV)
    cnt = torch.full((1,), -7, dtype=torch.int64, device=DEV)
    capi.check(L.apt_relabel_static(capi._ptr(seeds), ns, capi._ptr(ns_dev), capi._ptr(nbr), nn, stride,
                                    capi._ptr(uniq), capi._ptr(rel), capi._ptr(cnt), capi._stream()))
    return uniq, rel, cnt


def test_static_relabel_matches_workspace_relabel(orc, capi):
    rng = np.random.default_rng(17)
    limit = capi.lib().apt_relabel_static_max_items()
    assert limit == 1 << 21
    # Two calls in a row, the second smaller (then a few more shapes, all sharing the one array).  Small inputs
    # normally take the single-workgroup kernel with its table in LDS, which never touches the shared array:
    # that path is switched off here, so that every call below runs its passes over the array and would show
    # what an earlier, larger call left in it.
    _static(capi, *_case(rng, 2000, 30_000, 1 << 30))           # first use resolves the array's address
    torch.cuda.synchronize()
    capi.set_tuning("relabel_lds", 0)
    try:
        for ns, nn, id_range in [(67_584, 1_013_760, 111_000_000), (1024, 5120, 3000), (0, 0, 10), (5, 0, 10),
                                 (6144, 61_440, 50_000), (1 << 20, 1 << 20, 1 << 40), (1, 3, 2)]:
            seeds, nbr = _case(rng, ns, nn, id_range)
            want_u, want_r, want_n = capi.relabel(seeds, nbr)
            uniq = torch.full((ns + nn,), -7, dtype=torch.int64, device=DEV)
            rel = torch.full((nn,), -7, dtype=torch.int64, device=DEV)
            cnt = torch.full((1,), -7, dtype=torch.int64, device=DEV)
            torch.cuda.synchronize()
            # free device memory as the driver reports it (hipMemGetInfo): sees a hipMalloc made behind
            # torch's back, which torch.cuda.memory_allocated() would not
            free_before, reserved_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
            capi.check(capi.lib().apt_relabel_static(capi._ptr(seeds), ns, None, capi._ptr(nbr), nn, 0, capi._ptr(uniq),
                                                     capi._ptr(rel), capi._ptr(cnt), capi._stream()))
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before
            n = int(cnt.item())
            assert n == int(want_n)
            assert torch.equal(uniq[:n], want_u[:n]) and torch.equal(rel, want_r)
            assert bool((uniq[n:] == -7).all())                     # nothing written past the count
            if ns + nn <= 200_000:                                  # and both against the oracle
                ou, orl = orc.relabel(seeds.cpu().numpy(), nbr.cpu().numpy())
                assert np.array_equal(uniq[:n].cpu().numpy(), ou) and np.array_equal(rel.cpu().numpy(), orl)
            del uniq, rel, cnt
    finally:
        capi.set_tuning("relabel_lds", 1)
    # the LDS path (small inputs, default setting) gives the same answer and allocates nothing either
    seeds, nbr = _case(rng, 1024, 5120, 3000)
    want_u, want_r, want_n = capi.relabel(seeds, nbr)
    uniq, rel, cnt = _static(capi, seeds, nbr)
    n = int(cnt.item())
    assert n == int(want_n) and torch.equal(uniq[:n], want_u[:n]) and torch.equal(rel, want_r)
    # device-side seed count (the frontier of a later hop): only the first n * stride neighbours count
    seeds, nbr = _case(rng, 4000, 4000 * 10, 20_000)
    ns_dev = torch.tensor([2500], dtype=torch.int64, device=DEV)
    uniq, rel, cnt = _static(capi, seeds, nbr, ns_dev, 10)
    want_u, want_r, want_n = capi.relabel(seeds[:2500].contiguous(), nbr[:25_000].contiguous())
    n = int(cnt.item())
    assert n == int(want_n) and torch.equal(uniq[:n], want_u[:n]) and torch.equal(rel[:25_000], want_r)


def test_static_relabel_rejects_what_does_not_fit(capi):
    L = capi.lib()
    limit = L.apt_relabel_static_max_items()
    one = torch.full((1,), 5, dtype=torch.int64, device=DEV)
    p = capi._ptr(one)
    for ns, nn in [(limit, 1), (1, limit), (limit + 1, 0), (1 << 62, 1 << 62)]:
        rc = L.apt_relabel_static(p, ns, None, p, nn, 0, p, p, p, capi._stream())
        assert rc != 0 and b"maximum" in L.apt_last_error()
    assert L.apt_relabel_static(p, -1, None, p, 0, 0, p, p, p, capi._stream()) != 0
    assert L.apt_relabel_static(p, 1, None, p, 0, 0, p, p, None, capi._stream()) != 0
    torch.cuda.synchronize()
    assert int(one.item()) == 5                                  # a rejected call enqueues nothing
