"""HIP library vs CPU oracle through the C ABI, bit-exact (needs an MI355X)."""
import numpy as np
import pytest
import torch

from helpers import small_graph, special_graph

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    return t.cpu().numpy()


def _graphs(orc, capi, indptr, indices, **kw):
    og = orc.Graph(indptr, indices, **kw)
    dkw = {k: (dev(v) if isinstance(v, np.ndarray) else v) for k, v in kw.items()}
    return og, capi.Graph(dev(indptr), dev(indices), **dkw)


# ------------------------------------------------------------------ sampling
@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("fanout", [1, 5, 10, 15, 16, 17, 64, 65, 130])
def test_sampling_special_rows(orc, capi, replace, fanout):
    indptr, indices, degs = special_graph()
    og, dg = _graphs(orc, capi, indptr, indices)
    frontier = np.concatenate([np.arange(len(degs)), [-1, len(indptr) + 3, 5, 6, 6]])
    want_n, want_c = orc.sample_neighbors(og, frontier, fanout, replace, 42, 3)
    total = torch.zeros(1, dtype=torch.int64, device=DEV)
    got_n, got_c = capi.sample_neighbors(dg, dev(frontier), fanout, replace, 42, 3, out_total=total)
    assert np.array_equal(host(got_c), want_c)
    assert np.array_equal(host(got_n), want_n)
    assert int(total.item()) == int(want_c.sum())


@pytest.mark.parametrize("lanes", [0, 8, 16, 32, 64])
@pytest.mark.parametrize("replace", [False, True])
def test_sampling_random_graph_all_lane_groups(orc, capi, lanes, replace):
    indptr, indices = small_graph(20000, 16, seed=11)
    og, dg = _graphs(orc, capi, indptr, indices)
    rng = np.random.default_rng(lanes)
    frontier = rng.integers(0, 20000, size=70001)               # ragged: not a multiple of any tile
    capi.set_tuning("sample_lanes_per_row", lanes)
    try:
        for fanout, hop in [(5, 0), (10, 1), (15, 2)]:
            want_n, want_c = orc.sample_neighbors(og, frontier, fanout, replace, 7, hop)
            got_n, got_c = capi.sample_neighbors(dg, dev(frontier), fanout, replace, 7, hop)
            assert np.array_equal(host(got_c), want_c)
            assert np.array_equal(host(got_n), want_n)
    finally:
        capi.set_tuning("sample_lanes_per_row", 0)


@pytest.mark.parametrize("direct_rows", [2, 4])
def test_sampling_several_unstaged_rows_per_group(orc, capi, direct_rows):
    """Lane groups that resolve two or four rows themselves (no LDS staging): same rows as one row per group,
    alone and inside the fused driver with its rank-table bids."""
    from apt_amd.pipeline import MiniBatchPipeline
    indptr, indices = small_graph(20000, 30, seed=23)
    og, dg = _graphs(orc, capi, indptr, indices)
    frontier = np.random.default_rng(6).integers(0, 20000, size=30011)
    cnt = torch.tensor([25003], dtype=torch.int64, device=DEV)
    capi.set_tuning("sample_direct_rows", direct_rows)
    try:
        for fanout, replace in [(15, False), (7, True), (5, False)]:
            want_n, want_c = orc.sample_neighbors(og, frontier[:25003], fanout, replace, 9, 1)
            got_n, got_c = capi.sample_neighbors(dg, dev(frontier), fanout, replace, 9, 1, num_frontier_dev=cnt)
            assert np.array_equal(host(got_c)[:25003], want_c)
            assert np.array_equal(host(got_n)[:25003 * fanout], want_n)
        pipe = MiniBatchPipeline(dg, None, 512, [5, 10, 15], gather=False)
        for batch in range(3):
            seeds = np.random.default_rng(batch).integers(0, 20000, size=512)
            pipe.run(dev(seeds), 40 + batch)
            res = pipe.result()
            want_in, want_blocks = orc.sample_blocks(og, seeds, [5, 10, 15], False, 40 + batch)
            assert np.array_equal(host(res["input_nodes"]), want_in)
            for got, want in zip(res["blocks"], want_blocks):
                for k in ("neighbors", "relabeled", "counts"):
                    assert np.array_equal(host(got[k]), want[k]), k
    finally:
        capi.set_tuning("sample_direct_rows", 0)


@pytest.mark.parametrize("min_wg,max_blocks", [(0, 7), (1, 5), (3, 0), (1, 0)])
def test_sampling_launch_shapes(orc, capi, min_wg, max_blocks):
    """A small grid striding over many tiles, several rows per lane group (rows
    staged in LDS) and one row per group (resolved directly) give the same rows;
    fanouts below and above the 64 lanes of a wavefront."""
    indptr, indices = small_graph(20000, 30, seed=21)
    og, dg = _graphs(orc, capi, indptr, indices)
    frontier = np.random.default_rng(5).integers(0, 20000, size=30011)
    cnt = torch.tensor([25003], dtype=torch.int64, device=DEV)
    capi.set_tuning("sample_min_workgroups", min_wg)
    capi.set_tuning("sample_max_blocks", max_blocks)
    try:
        for fanout, replace in [(15, False), (7, True), (100, False), (70, True)]:
            want_n, want_c = orc.sample_neighbors(og, frontier[:25003], fanout, replace, 9, 1)
            got_n, got_c = capi.sample_neighbors(dg, dev(frontier), fanout, replace, 9, 1, num_frontier_dev=cnt)
            assert np.array_equal(host(got_c)[:25003], want_c)
            assert np.array_equal(host(got_n)[:25003 * fanout], want_n)
    finally:
        capi.set_tuning("sample_min_workgroups", 0)
        capi.set_tuning("sample_max_blocks", 0)


def test_sampling_position_map_and_partition(orc, capi):
    indptr, indices = small_graph(5000, 12, seed=12)
    n = 5000
    cached = np.arange(0, n, 7)
    c_indptr = np.zeros(len(cached) + 1, dtype=np.int64)
    c_indptr[1:] = np.cumsum(indptr[cached + 1] - indptr[cached])
    c_indices = np.concatenate([indices[indptr[v]:indptr[v + 1]] for v in cached])
    pos = -np.arange(n, dtype=np.int64) - 2
    pos[cached] = np.arange(len(cached))
    og, dg = _graphs(orc, capi, indptr, indices, cached_indptr=c_indptr, cached_indices=c_indices,
                     adj_pos_map=pos)
    f = np.random.default_rng(0).integers(-2, n + 10, size=9000)
    for replace in (False, True):
        want = orc.sample_neighbors(og, f, 6, replace, 3, 0)
        got = capi.sample_neighbors(dg, dev(f), 6, replace, 3, 0)
        assert np.array_equal(host(got[0]), want[0]) and np.array_equal(host(got[1]), want[1])
    og, dg = _graphs(orc, capi, indptr[1000:3001] - indptr[1000],
                     indices[indptr[1000]:indptr[3000]], row_begin=1000)
    want = orc.sample_neighbors(og, f, 6, False, 3, 0)
    got = capi.sample_neighbors(dg, dev(f), 6, False, 3, 0)
    assert np.array_equal(host(got[0]), want[0]) and np.array_equal(host(got[1]), want[1])


def test_sampling_device_side_count_and_empty(orc, capi):
    indptr, indices = small_graph(3000, 10, seed=13)
    og, dg = _graphs(orc, capi, indptr, indices)
    f = np.arange(3000)
    cnt = torch.tensor([1234], dtype=torch.int64, device=DEV)
    out = torch.full((3000 * 4,), -7, dtype=torch.int64, device=DEV)
    capi.sample_neighbors(dg, dev(f), 4, False, 1, 0, num_frontier_dev=cnt, out_neighbors=out)
    want, _ = orc.sample_neighbors(og, f[:1234], 4, False, 1, 0)
    o = host(out)
    assert np.array_equal(o[:1234 * 4], want) and np.all(o[1234 * 4:] == -7)
    e = capi.sample_neighbors(dg, dev(np.array([], dtype=np.int64)), 4, False, 1, 0)
    assert e[0].numel() == 0 and e[1].numel() == 0


def test_sampling_bad_arguments(capi):
    indptr, indices = small_graph(100, 4, seed=1)
    dg = capi.Graph(dev(indptr), dev(indices))
    with pytest.raises(capi.AptError):
        capi.sample_neighbors(dg, dev(np.arange(4)), 0, False, 1, 0)
    with pytest.raises(capi.AptError):
        capi.sample_neighbors(dg, dev(np.arange(4)), 5000, False, 1, 0)
    with pytest.raises(TypeError):
        capi.sample_neighbors(dg, torch.arange(4), 3, False, 1, 0)          # CPU tensor
    with pytest.raises(TypeError):
        capi.sample_neighbors(dg, torch.arange(4, device=DEV, dtype=torch.int32), 3, False, 1, 0)


# ------------------------------------------------------------------ relabel
def _relabel_case(orc, capi, seeds, nbrs):
    want_u, want_r = orc.relabel(seeds, nbrs)
    u, r, n = capi.relabel(dev(np.asarray(seeds, np.int64)), dev(np.asarray(nbrs, np.int64)))
    assert n == len(want_u)
    assert np.array_equal(host(u), want_u)
    assert np.array_equal(host(r), want_r)


def test_relabel_random_sizes(orc, capi):
    rng = np.random.default_rng(0)
    for ns, f, hi in [(1, 1, 5), (10, 3, 20), (1024, 5, 3000), (6144, 10, 100000),
                      (67584, 15, 2_400_000), (1023, 1, 1 << 40)]:
        seeds = rng.permutation(min(hi, 10_000_000))[:ns].astype(np.int64)
        nbrs = rng.integers(0, hi, size=ns * f)
        _relabel_case(orc, capi, seeds, nbrs)


def test_relabel_equal_tags_and_reversed_duplicates(orc, capi):
    """Different ids whose 32-bit table tags are equal (the tag only filters; the
    id itself decides), and duplicates laid out so that later items tend to reach
    the table first (a word is then lowered and its item displaced)."""
    C2 = 0xD6E8FEB86659FD93
    inv = pow(C2, -1, 1 << 64)
    same_tag = [t * inv % (1 << 64) for t in range(1, 4000)]
    same_tag = np.array([0] + [d for d in same_tag if d < (1 << 62)][:700], dtype=np.int64)
    assert len({(int(k) * C2 % (1 << 64)) >> 32 for k in same_tag}) == 1 and len(same_tag) > 300
    rng = np.random.default_rng(9)
    nbrs = same_tag[rng.integers(0, len(same_tag), size=5000)]
    _relabel_case(orc, capi, same_tag[:100][::-1].copy(), nbrs)
    # every id many times, spread over the whole item range
    ids = rng.permutation(5000)[:2000].astype(np.int64)
    _relabel_case(orc, capi, ids[:256], np.tile(ids, 300))


def test_relabel_specials(orc, capi):
    rng = np.random.default_rng(1)
    e = np.array([], dtype=np.int64)
    _relabel_case(orc, capi, np.array([5, 9, 7]), e)
    _relabel_case(orc, capi, e, np.array([3, 3, 1, 3]))
    _relabel_case(orc, capi, e, e)
    _relabel_case(orc, capi, np.array([4]), np.full(5000, 4))
    _relabel_case(orc, capi, np.array([2, 2, 8, 2]), np.array([8, 1, 2, 1]))
    _relabel_case(orc, capi, np.arange(512), rng.integers(0, 512, 512))
    _relabel_case(orc, capi, np.arange(1024), rng.integers(0, 1024, 1024 * 3))
    big = 111_059_956
    _relabel_case(orc, capi, np.array([big - 1, 0, big - 2]), rng.integers(big - 50, big, 640))
    _relabel_case(orc, capi, np.arange(8) * 4096, rng.integers(0, 8, 1000) * 4096)
    _relabel_case(orc, capi, np.array([3, 1]), np.array([1, -1, 7, -1, 3]))
    # heavy duplication (hub ids) in a large list
    hubs = rng.integers(0, 50, size=300000)
    tail = rng.integers(0, 5_000_000, size=300000)
    _relabel_case(orc, capi, rng.permutation(5_000_000)[:4096], rng.permutation(np.concatenate([hubs, tail])))


def test_relabel_ranked_fresh_and_continued(orc, capi):
    """apt_relabel_ranked (node-indexed rank table) against the oracle: fresh calls with repeated seeds, padding,
    heavy duplication, ids at the table's end; chains of calls where each call's seeds are the unique list of the
    one before (the reference's per-hop pattern), which continue the batch in the table; ids beyond the table."""
    rng = np.random.default_rng(3)
    N = 2_000_000
    rr = capi.RankedRelabel(N, DEV)
    e = np.array([], dtype=np.int64)
    cases = [(np.array([5, 9, 7]), e), (e, np.array([3, 3, 1, 3])), (e, e), (np.array([4]), np.full(5000, 4)),
             (np.array([2, 2, 8, 2]), np.array([8, 1, 2, 1])), (np.array([3, 1]), np.array([1, -1, 7, -1, 3])),
             (np.array([N - 1, 0, N - 2]), rng.integers(N - 50, N, 640)),
             (rng.permutation(N)[:4096], rng.permutation(np.concatenate([rng.integers(0, 50, 300000),
                                                                         rng.integers(0, N, 300000)]))),
             (rng.integers(0, 1000, 3000), np.where(rng.random(50000) < 0.2, -1, rng.integers(0, 3000, 50000)))]
    for seeds, nbrs in cases + cases[:3]:                        # again: the table is reused without clearing
        seeds, nbrs = np.asarray(seeds, np.int64), np.asarray(nbrs, np.int64)
        u, r, n = rr.relabel(dev(seeds), dev(nbrs))
        want_u, want_r = orc.relabel(seeds, nbrs)
        assert n == len(want_u) and np.array_equal(host(u), want_u) and np.array_equal(host(r), want_r)
    # chains: hop h's seeds are hop h-1's unique list
    for chain in range(4):
        frontier = dev(rng.integers(0, N, 700))                  # repeated seeds happen
        first = True
        for f in (5, 10, 15):
            nbrs = np.where(rng.random(frontier.numel() * f) < 0.1, -1, rng.integers(0, N if chain % 2 else 30000,
                                                                                      frontier.numel() * f))
            want_u, want_r = orc.relabel(host(frontier), nbrs)
            assert first or rr._last == (frontier.data_ptr(), frontier.numel(), frontier._version)
            u, r, n = rr.relabel(frontier, dev(nbrs))
            assert n == len(want_u) and np.array_equal(host(u), want_u) and np.array_equal(host(r), want_r)
            frontier, first = u, False
    # a seeds tensor that was modified in place, or is another tensor with the same values, starts afresh
    u, r, n = rr.relabel(dev(np.arange(100, 9100)), dev(rng.integers(0, N, 40000)))
    v = u.clone()
    nbrs = rng.integers(0, N, 60000)
    want_u, want_r = orc.relabel(host(v), nbrs)
    u2, r2, _ = rr.relabel(v, dev(nbrs))
    assert np.array_equal(host(u2), want_u) and np.array_equal(host(r2), want_r)
    u2[5:7] = u2[5:7].flip(0)                                    # in-place edit: the version changes
    assert rr._last != (u2.data_ptr(), u2.numel(), u2._version)
    want_u, want_r = orc.relabel(host(u2), nbrs)
    u3, r3, _ = rr.relabel(u2, dev(nbrs))
    assert np.array_equal(host(u3), want_u) and np.array_equal(host(r3), want_r)
    # an id the table cannot hold is reported, not mislabelled
    with pytest.raises(capi.AptError, match="outside"):
        rr.relabel(dev(np.array([1, 2, N])), dev(np.array([3, 4])))
    with pytest.raises(capi.AptError, match="outside"):
        rr.relabel(dev(np.array([1, 2])), dev(np.array([3, N + 7, 4])))
    u, r, n = rr.relabel(dev(np.array([1, 2])), dev(np.array([3, 2, 4])))     # and the table is usable afterwards
    assert host(u).tolist() == [1, 2, 3, 4] and host(r).tolist() == [2, 1, 3]
    # device-side count and stride (the per-hop driver's form), fresh and continued
    cap, f, real = 5000, 5, 3210
    seeds, nbrs = rng.permutation(100000)[:cap], rng.integers(0, 100000, size=cap * f)
    cnt = torch.tensor([real], dtype=torch.int64, device=DEV)
    uq = torch.full((cap * (f + 1),), -7, dtype=torch.int64, device=DEV)
    rl = torch.full((cap * f,), -7, dtype=torch.int64, device=DEV)
    counts = torch.zeros(2, dtype=torch.int64, device=DEV)
    rr.enqueue(dev(seeds), dev(nbrs), False, uq, rl, counts[0:1], counts[1:2], num_seeds_dev=cnt, neighbor_stride=f)
    want_u, want_r = orc.relabel(seeds[:real], nbrs[:real * f])
    assert host(counts).tolist() == [len(want_u), 0]
    assert np.array_equal(host(uq)[:len(want_u)], want_u) and np.array_equal(host(rl)[:real * f], want_r)
    nb2 = rng.integers(0, 100000, size=uq.numel() * 3)
    uq2 = torch.full((uq.numel() * 4,), -7, dtype=torch.int64, device=DEV)
    rl2 = torch.full((uq.numel() * 3,), -7, dtype=torch.int64, device=DEV)
    n1 = counts[0:1].clone()
    rr.enqueue(uq, dev(nb2), True, uq2, rl2, counts[0:1], counts[1:2], num_seeds_dev=n1, neighbor_stride=3)
    want_u2, want_r2 = orc.relabel(want_u, nb2[:len(want_u) * 3])
    assert host(counts).tolist() == [len(want_u2), 0]
    assert np.array_equal(host(uq2)[:len(want_u2)], want_u2) and np.array_equal(host(rl2)[:len(want_u) * 3], want_r2)


def test_relabel_device_side_count(orc, capi):
    rng = np.random.default_rng(2)
    cap, f, real = 5000, 5, 3210
    seeds = rng.permutation(100000)[:cap]
    nbrs = rng.integers(0, 100000, size=cap * f)
    cnt = torch.tensor([real], dtype=torch.int64, device=DEV)
    u, r, nu = capi.relabel(dev(seeds), dev(nbrs), num_seeds_dev=cnt, neighbor_stride=f, sync=False)
    want_u, want_r = orc.relabel(seeds[:real], nbrs[:real * f])
    n = int(nu.item())
    assert n == len(want_u)
    assert np.array_equal(host(u)[:n], want_u)
    assert np.array_equal(host(r)[:real * f], want_r)


def test_relabel_lds_path_and_table_path(orc, capi):
    """Inputs of up to 8192 items are relabelled by one workgroup with its table in LDS, larger ones by
    the passes over a table in device memory; both against the oracle on the same small inputs (the
    switch selects the path), at the size limit, with keys that collide in the LDS table, with padding
    and with a device-side count."""
    rng = np.random.default_rng(5)
    G = 0x9E3779B97F4A7C15
    inv = pow(G, -1, 1 << 64)
    # keys whose LDS slot (top 14 bits of key * G) is the same: one long probe chain
    chain = np.array([k for k in ((t * inv) % (1 << 64) for t in range(1, 3000)) if k < (1 << 62)][:900],
                     dtype=np.int64)
    assert len({(int(k) * G % (1 << 64)) >> 50 for k in chain}) == 1 and len(chain) > 500
    cases = [
        (rng.permutation(50_000)[:1024], rng.integers(0, 50_000, 1024 * 7)),             # 8192 items: the limit
        (rng.permutation(50_000)[:1024], rng.integers(0, 50_000, 1024 * 7 + 1)),         # one more: table path
        (np.arange(8192), np.array([], dtype=np.int64)),                                 # all distinct, table half full
        (np.array([], dtype=np.int64), np.full(8192, 7)),                                # one key 8192 times
        (chain[:64][::-1].copy(), chain[rng.integers(0, len(chain), 6000)]),
        (np.array([5, -1, 5, 9]), np.where(rng.random(4000) < 0.3, -1, rng.integers(0, 60, 4000))),
        (rng.integers(0, 1 << 40, 100), rng.integers(0, 1 << 40, 3000)),
        (np.array([111_059_955, 0]), rng.integers(111_059_900, 111_059_956, 700)),
    ]
    try:
        for lds in (1, 0):
            capi.set_tuning("relabel_lds", lds)
            for seeds, nbrs in cases:
                _relabel_case(orc, capi, np.asarray(seeds, np.int64), np.asarray(nbrs, np.int64))
            # device-side count on a small plan (first hop of a batch of 1024 at fanout 5)
            seeds, nbrs = rng.permutation(100_000)[:1024], rng.integers(0, 100_000, 1024 * 5)
            cnt = torch.tensor([700], dtype=torch.int64, device=DEV)
            u, r, nu = capi.relabel(dev(seeds), dev(nbrs), num_seeds_dev=cnt, neighbor_stride=5, sync=False)
            want_u, want_r = orc.relabel(seeds[:700], nbrs[:3500])
            n = int(nu.item())
            assert n == len(want_u) and np.array_equal(host(u)[:n], want_u) and np.array_equal(host(r)[:3500], want_r)
    finally:
        capi.set_tuning("relabel_lds", 1)


# ------------------------------------------------------------------ gather
def _rand_table(rng, rows, dim, dtype):
    if dtype == torch.float32:
        return rng.standard_normal((rows, dim)).astype(np.float32)
    return rng.integers(0, 65535, size=(rows, dim)).astype(np.uint16)   # raw 16-bit patterns


def _to_dev_table(a, dtype):
    t = torch.from_numpy(a.view(np.int16) if a.dtype == np.uint16 else a).to(DEV)
    return t.view(dtype) if a.dtype == np.uint16 else t


@pytest.mark.parametrize("dtype,dim", [(torch.float32, 128), (torch.float32, 100), (torch.bfloat16, 128),
                                       (torch.float32, 7), (torch.bfloat16, 5), (torch.float32, 256),
                                       (torch.float32, 602), (torch.bfloat16, 1024), (torch.float32, 2)])
@pytest.mark.parametrize("rows_in_flight", [0, 1, 8])
def test_gather_identity_map(orc, capi, dtype, dim, rows_in_flight):
    rng = np.random.default_rng(dim)
    table = _rand_table(rng, 5000, dim, dtype)
    idx = np.concatenate([rng.integers(0, 5000, size=20011), [-1, 5000, 4999, 0]])
    want, wmiss = orc.gather_rows(orc.FeatStore(table), idx)
    capi.set_tuning("gather_rows_in_flight", rows_in_flight)
    try:
        miss = torch.zeros(1, dtype=torch.int64, device=DEV)
        st = capi.FeatStore(_to_dev_table(table, dtype))
        out = capi.gather_rows(st, dev(idx), miss_count=miss)
    finally:
        capi.set_tuning("gather_rows_in_flight", 0)
    got = host(out.view(torch.int16) if dtype == torch.bfloat16 else out)
    assert np.array_equal(got.view(want.dtype), want)
    assert int(miss.item()) == wmiss == 2


@pytest.mark.parametrize("D,Dr,off", [(128, 128, 0), (128, 32, 64), (24, 8, 12), (25, 7, 3), (100, 50, 50)])
def test_gather_two_tables(orc, capi, D, Dr, off):
    rng = np.random.default_rng(D + off)
    total, nloc, ncache = 20000, 6000, 1500
    local = rng.standard_normal((nloc, D)).astype(np.float32)
    cache = rng.standard_normal((ncache, Dr)).astype(np.float32)
    local_idx = rng.permutation(total)[:nloc]
    cached_idx = np.concatenate([local_idx[:700], np.setdiff1d(np.arange(total), local_idx)[:800]])
    pos = np.full(total, -1, dtype=np.int64)
    pos[local_idx] = -np.arange(nloc) - 2
    pos[cached_idx] = np.arange(ncache)
    idx = np.concatenate([rng.integers(0, total, 30000), [-1, total, total + 7]])
    want, wmiss = orc.gather_rows(orc.FeatStore(local, cache, pos, col_offset=off, out_dim=Dr), idx)
    miss = torch.zeros(1, dtype=torch.int64, device=DEV)
    st = capi.FeatStore(dev(local), dev(cache), dev(pos), col_offset=off, out_dim=Dr)
    out = capi.gather_rows(st, dev(idx), miss_count=miss)
    assert np.array_equal(host(out), want)
    assert int(miss.item()) == wmiss


def test_gather_empty_and_device_count(orc, capi):
    rng = np.random.default_rng(9)
    table = rng.standard_normal((1000, 64)).astype(np.float32)
    st = capi.FeatStore(dev(table))
    assert capi.gather_rows(st, dev(np.array([], dtype=np.int64))).shape == (0, 64)
    idx = rng.integers(0, 1000, 4000)
    cnt = torch.tensor([2500], dtype=torch.int64, device=DEV)
    out = torch.full((4000, 64), 5.0, device=DEV)
    capi.gather_rows(st, dev(idx), num_index_dev=cnt, out=out)
    o = host(out)
    assert np.array_equal(o[:2500], table[idx[:2500]]) and np.all(o[2500:] == 5.0)


def test_gather_store_rules_give_the_same_rows(capi):
    """An output above 128 MB is stored non-temporal except for its end, which goes write-through (how much is a
    knob); whatever the split, and with every forced policy, the rows are those of torch's index_select.  The
    device-side count decides where the end is."""
    from apt_amd import synth
    n_rows, D, n = 1_000_000, 128, 600_000                       # 600 k rows of 256 B: 154 MB
    feats = synth.random_features(n_rows, D, torch.bfloat16, 4, DEV)
    idx = torch.randint(0, n_rows, (n,), device=DEV)
    want = feats.index_select(0, idx).view(torch.int16)
    fs = capi.FeatStore(feats)
    n_dev = torch.tensor([n - 12_345], device=DEV)
    try:
        for policy, tail in ((0, 0), (0, 1), (0, 32), (0, 1024), (1, 0), (2, 0), (3, 0)):
            capi.set_tuning("gather_store_policy", policy)
            capi.set_tuning("gather_wt_tail_mib", tail)
            out = capi.gather_rows(fs, idx)
            assert torch.equal(out.view(torch.int16), want), (policy, tail)
            out = torch.zeros_like(out)
            capi.gather_rows(fs, idx, num_index_dev=n_dev, out=out)
            k = int(n_dev.item())
            assert torch.equal(out[:k].view(torch.int16), want[:k]) and not out[k:].any(), (policy, tail)
    finally:
        capi.set_tuning("gather_store_policy", 0)
        capi.set_tuning("gather_wt_tail_mib", 0)


def test_permute_scatter_rows(orc, capi):
    rng = np.random.default_rng(10)
    for dim, dtype in [(16, torch.float32), (256, torch.float32), (64, torch.bfloat16), (3, torch.float32)]:
        x = _rand_table(rng, 4321, dim, dtype)
        perm = rng.permutation(4321)
        xd = _to_dev_table(x, dtype)
        up = capi.permute_rows(xd, dev(perm))
        pk = capi.scatter_rows(xd, dev(perm))
        as_np = lambda t: host(t.view(torch.int16) if dtype == torch.bfloat16 else t).view(x.dtype)
        assert np.array_equal(as_np(up), orc.permute_rows(x, perm))
        assert np.array_equal(as_np(pk), orc.scatter_rows(x, perm))
        assert np.array_equal(as_np(capi.permute_rows(pk, dev(perm))), x)       # round trip
    # pack into more rows than are named (some ids out of range): the rows nobody names come back zero,
    # on memory that held something else before
    for dim, dtype in [(5, torch.float32), (256, torch.float32), (7, torch.bfloat16), (64, torch.bfloat16)]:
        x = _rand_table(rng, 3000, dim, dtype)
        dest = rng.permutation(5000)[:3000]
        dest[[4, 77]] = [-1, 5000]
        junk = torch.full((5000, dim), 3.0, device=DEV).to(dtype)     # recycled by the allocator below
        del junk
        pk = capi.scatter_rows(_to_dev_table(x, dtype), dev(dest), num_out_rows=5000)
        as_np = lambda t: host(t.view(torch.int16) if dtype == torch.bfloat16 else t).view(x.dtype)
        want = np.zeros((5000, dim), dtype=x.dtype)
        ok = (dest >= 0) & (dest < 5000)
        want[dest[ok]] = x[ok]
        assert np.array_equal(as_np(pk), want), (dim, dtype)
    # un-unique gather: more outputs than inputs
    inv = rng.integers(0, 100, size=999)
    x = rng.standard_normal((100, 32)).astype(np.float32)
    assert np.array_equal(host(capi.permute_rows(dev(x), dev(inv))), x[inv])


# ------------------------------------------------------------------ bucketing
def test_cluster_permute_reference_fixture(orc, capi):
    for W in (1, 2, 4, 8):
        for rank in range(W):
            min_vids = 100 * np.arange(W + 1)
            seeds = W * np.arange(99) + rank
            want = orc.cluster_permute(seeds, min_vids, W, 0, rank, 0, W)
            got = capi.cluster_permute(dev(seeds), dev(min_vids), W, 0, rank, 0, W)
            for g, w in zip(got, want):
                assert np.array_equal(host(g), w)


def test_cluster_permute_random(orc, capi):
    rng = np.random.default_rng(5)
    for W, n in [(8, 5000), (8, 1_080_000), (33, 70001), (64, 12345), (1, 1000), (8, 0)]:
        min_vids = np.concatenate([[0], np.sort(rng.integers(1, 10**7, W - 1)), [10**7]]).astype(np.int64)
        ids = rng.integers(0, 10**7, size=n)
        for (off, rank, beg, end) in [(0, 0, 0, W), (0, W // 2, W // 2, W), (min(2, W - 1), 0, 0, W)]:
            want = orc.cluster_permute(ids, min_vids, W, off, rank, beg, end)
            got = capi.cluster_permute(dev(ids), dev(min_vids), W, off, rank, beg, end)
            for g, w in zip(got, want):
                assert np.array_equal(host(g), w)


def test_cluster_reqs(orc, capi):
    rng = np.random.default_rng(6)
    W, R, total = 8, 4, 200000
    min_vids = np.arange(W + 1) * (total // W)
    fm = np.where(rng.random(total) < 0.4, -1, rng.integers(-5000, 5000, total)).astype(np.int64)
    rwm = np.array([0, 0, 1, 1, 2, 2, 3, 3])
    ids = rng.integers(0, total, size=300000)
    want = orc.cluster_reqs(ids, fm, rwm, min_vids, W, R)
    got = capi.cluster_reqs(dev(ids), dev(fm), dev(rwm), dev(min_vids), W, R)
    for g, w in zip(got, want):
        assert np.array_equal(host(g), w)


# ------------------------------------------------------------------ uniformity on the GPU itself
@pytest.mark.parametrize("deg,fanout,replace", [(16, 15, False), (40, 10, False), (1000, 15, False),
                                                (37, 8, True), (6, 3, False)])
def test_sampling_uniformity_chi_square(capi, deg, fanout, replace):
    """20000 nodes with identical rows 0..deg-1: every node is an independent
    draw (the counter is keyed by the node id), so the position histogram must
    be flat; for deg=6, k=3 all 20 subsets must be equally likely."""
    import itertools
    from scipy import stats
    n = 20000
    indptr = np.arange(n + 1, dtype=np.int64) * deg
    indices = np.tile(np.arange(deg, dtype=np.int64), n)
    dg = capi.Graph(dev(indptr), dev(indices))
    nbr, cnt = capi.sample_neighbors(dg, dev(np.arange(n)), fanout, replace, 987654321, 2)
    nbr = host(nbr).reshape(n, fanout)
    assert np.all(host(cnt) == fanout) and nbr.min() >= 0 and nbr.max() < deg
    hist = np.bincount(nbr.reshape(-1), minlength=deg)
    assert stats.chisquare(hist).pvalue > 1e-4
    if not replace:
        assert all(len(set(r.tolist())) == fanout for r in nbr[:2000])        # distinct positions
        if deg == 6:
            subsets = {s: 0 for s in itertools.combinations(range(deg), fanout)}
            for r in nbr:
                subsets[tuple(sorted(r.tolist()))] += 1
            obs = np.array(list(subsets.values()))
            assert np.all(obs > 0) and stats.chisquare(obs).pvalue > 1e-4
    else:
        for s in range(fanout):                                               # every slot on its own
            assert stats.chisquare(np.bincount(nbr[:, s], minlength=deg)).pvalue > 1e-5
