"""The C ABI from plain C: tests/c_abi/epoch_consumer.c (built with gcc by apt_amd/build.py, no Python or torch in
it) runs two epochs through the library's epoch driver and checks every batch itself; its totals must be what the
Python pipeline gets for the same graph, seeds and keys."""
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "c_abi", "epoch_consumer")


def test_c_consumer_is_built():
    assert os.path.exists(BINARY), "tests/c_abi/epoch_consumer is missing: run apt_amd/build.py"


@pytest.mark.gpu
def test_c_consumer_matches_python_pipeline(capi):
    import torch

    from apt_amd.pipeline import MiniBatchPipeline
    r = subprocess.run([BINARY], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout[-1000:] + r.stderr[-3000:]
    m = re.search(r"ok batches=(\d+) edges=(\d+) nodes=(\d+) checksum=(\d+)", r.stdout)
    assert m, r.stdout
    got = tuple(int(x) for x in m.groups())
    # the same graph, features, seeds and keys as the program's
    N, DIM, B, hops, batches = 20000, 16, 192, [4, 3], 9
    deg = 3 + np.arange(N) % 9
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    v = np.repeat(np.arange(N), deg)
    k = np.arange(indptr[-1]) - indptr[v]
    indices = ((v * 7 + k * 1301 + 1) % N).astype(np.int64)
    g = capi.Graph(torch.from_numpy(indptr).cuda(), torch.from_numpy(indices).cuda())
    feats = torch.arange(N * DIM, dtype=torch.float32, device="cuda").view(N, DIM)
    pipe = MiniBatchPipeline(g, capi.FeatStore(feats), B, hops)
    edges = nodes = checksum = 0
    for epoch in range(2):
        seeds = (np.arange(batches * B) * 97 + epoch * 31) % N
        for i in range(batches):
            pipe.run(torch.from_numpy(seeds[i * B:(i + 1) * B]).cuda(), 1000 * (epoch + 1) + i)
            res = pipe.result()
            edges += res["num_edges"]
            nodes += res["input_nodes"].numel()
            checksum += int(res["input_nodes"].sum())
            assert torch.equal(res["features"], feats[res["input_nodes"]])
    assert got == (2 * batches, edges, nodes, checksum)
