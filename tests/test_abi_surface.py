"""No-GPU checks of the drop-in boundary: the C-ABI library exports every
symbol the headers declare, and the torch operator library registers the
operator names (and inferred schemas) the reference binds."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions(hdr):
    text = open(os.path.join(ROOT, "include", hdr)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(apt_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from apt_amd import capi
    for hdr, path, table, least in (("apt_amd.h", capi.LIB_PATH, capi.SYMBOLS, 15),
                                    ("apt_synth.h", capi.BENCH_LIB_PATH, capi.BENCH_SYMBOLS, 4)):
        lib = ctypes.CDLL(path)
        declared = _declared_functions(hdr)
        assert len(declared) >= least
        for name in declared:
            assert hasattr(lib, name), f"{name} declared in include/{hdr} but not exported by {path}"
            assert name in table, f"{name} has no ctypes prototype in capi"
        assert sorted(table) == declared, f"capi binds symbols that include/{hdr} does not declare"
    version = int(re.search(r"#define APT_ABI_VERSION (\d+)", open(os.path.join(ROOT, "include", "apt_amd.h")).read()).group(1))
    assert capi.lib().apt_abi_version() == version == capi.ABI_VERSION
    capi.bench_lib()


def test_product_library_exports_the_product_abi_only():
    """Benchmark inputs and probes live in libapt_bench.so: the product library exports what
    include/apt_amd.h declares and nothing named apt_synth_*."""
    import subprocess

    from apt_amd import capi
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line and line.split()[-1].startswith("apt_")}
    assert exported == set(_declared_functions("apt_amd.h")), exported ^ set(_declared_functions("apt_amd.h"))


def test_argument_checks_need_no_gpu():
    """Host-side validation runs before anything touches the device."""
    from apt_amd import capi
    L = capi.lib()
    g = capi.CGraph()
    assert L.apt_sample_neighbors(ctypes.byref(g), None, -1, None, 5, 0, 1, 0, None, None, None, None) != 0
    assert b"num_frontier" in L.apt_last_error()
    assert L.apt_sample_neighbors(ctypes.byref(g), None, 4, None, 0, 0, 1, 0, None, None, None, None) != 0
    assert b"fanout" in L.apt_last_error()
    assert L.apt_relabel(None, -1, None, None, 0, 0, None, None, None, None, None, 0, None) != 0
    assert L.apt_relabel_workspace_bytes(1 << 40) == 0
    assert L.apt_relabel_workspace_bytes(1000) > 0
    assert L.apt_bucket_workspace_bytes(10, 0) == 0 and L.apt_bucket_workspace_bytes(10, 8) > 0
    assert L.apt_set_tuning(b"no_such_knob", 1) != 0
    fan = (ctypes.c_int * 3)(5, 10, 15)
    assert L.apt_minibatch_capacity(4096, fan, 3, 3) == 4096 * 6 * 11 * 16
    assert L.apt_minibatch_capacity(1 << 28, fan, 3, 3) == -1          # ids would not fit 32 bits
    assert L.apt_rank_table_bytes(111_059_956) >= 4 * 111_059_956
    # entry points added around the core path
    assert L.apt_block_workspace_bytes(1000, 15, 5000, 1) > L.apt_block_workspace_bytes(1000, 15, 5000, 0) > 0
    assert L.apt_block_workspace_bytes(1 << 40, 15, 5000, 1) == 0
    assert L.apt_block_formats(None, 10, None, 5, 100, None, None, None, None, None, None, None, None, 0, None) != 0
    assert b"csc_indptr" in L.apt_last_error()
    assert L.apt_count_ids(None, -1, None, None, 10, None) != 0
    assert L.apt_csr_copy_rows(None, None, 0, None, 5, None, 7, None, None) != 0
    assert L.apt_gat_block(None, 10, None, 0, None, 5, 4, 64, 2, None, None, 0.2, None, None, None) != 0
    assert b"fanout" in L.apt_last_error()
    assert L.apt_gat_scores(None, 10, 4, 64, 3, None, None, None) != 0 and b"elem_size" in L.apt_last_error()
    assert L.apt_map_to_vir(None, 5, None, 10, 0, None, 8, 0, 0, 0, 8, None, None) != 0
    assert L.apt_vir_send_offset(0, 5, None, 0, None, 0, 0, None, None) != 0
    assert L.apt_spmm_block(None, 5, None, 0, None, 5, 8, 4, 0, None, None) != 0
    assert L.apt_coo_is_grouped(None, 5, None, None) != 0
    assert L.apt_scatter_workspace_bytes(64) == 68 and L.apt_scatter_workspace_bytes(65) == 72
    assert L.apt_scatter_rows(None, None, 3, 8, 4, None, 5, None, 0, None) != 0
    assert L.apt_spmm_heads(None, None, 5, None, 5, None, None, 3, 8, 4, 1, None, 5, None, None, None, None) != 0
    assert b"heads" in L.apt_last_error()
    for key in (b"sample_min_workgroups", b"gather_vector_bytes", b"block_fused_scan"):
        assert L.apt_set_tuning(key, 0) == 0
    assert L.apt_set_tuning(b"block_fused_scan", 1) == 0
    assert L.apt_set_tuning(b"gather_vector_bytes", 3) != 0
    for key in (b"relabel_lds",):
        assert L.apt_set_tuning(key, 0) == 0 and L.apt_set_tuning(key, 1) == 0
    assert L.apt_set_tuning(b"gather_wt_tail_mib", 64) == 0 and L.apt_set_tuning(b"gather_wt_tail_mib", 0) == 0
    assert L.apt_set_tuning(b"gather_wt_tail_mib", -1) != 0
    assert L.apt_time_next_gather(None, None) == 0
    blank = (ctypes.c_uint64 * 64)()
    assert L.apt_minibatch_lookup(ctypes.addressof(blank), None) != 0 and b"pending" in L.apt_last_error()
    assert L.apt_minibatch_lookup(None, None) != 0
    assert L.apt_gather_rows_with_lookup(None, None, 0, None, None, None, None, None) != 0


REFERENCE_OPS = {   # reference src/pybind.cc:19-47 with the schemas torch infers from the C++ types
    "nccl_get_unique_id": "() -> Tensor",
    "init": "(int _0, int _1, int _2, Tensor _3, int _4) -> ()",
    "cache_feats_shared": "(int _0, Tensor _1, Tensor _2, Tensor _3, Tensor _4, int _5) -> ()",
    "mix_cache_graphs": "(int _0, Tensor _1, Tensor _2, Tensor _3, Tensor _4, Tensor _5) -> ()",
    "register_min_vids": "(Tensor _0, int _1) -> ()",
    "register_multi_machines_scheme": "(Tensor _0, Tensor _1) -> ()",
    "cpu_load_subtensor": "(Tensor _0) -> Tensor",
    "load_subtensor": "(Tensor _0) -> Tensor",
    "crossmachine_load_subtensor": "(Tensor _0) -> Tensor",
    "cluster_reqs": "(Tensor _0) -> (Tensor, Tensor, Tensor)",
    "local_sample_one_layer": "(Tensor _0, int _1) -> Tensor[]",
    "np_sample_and_shuffle": "(Tensor _0, int _1) -> Tensor[]",
    "feat_shuffle": "(Tensor _0, Tensor _1, Tensor _2, Tensor _3, int _4, int _5) -> Tensor",
    "shuffle_seeds": "(Tensor _0) -> (Tensor, Tensor, Tensor, Tensor)",
    "relabel_csc": "(Tensor _0, Tensor _1) -> Tensor[]",
    "srcdst_to_vir": "(int _0, Tensor _1, Tensor _2) -> Tensor",
    "src_to_vir": "(int _0, int _1, Tensor _2) -> Tensor",
    "spmm_copy_u_sum": "(Tensor _0, Tensor _1, Tensor _2, Tensor _3, Tensor _4, Tensor _5) -> Tensor",
    "spmm_copy_e_sum": "(Tensor _0, Tensor _1, Tensor _2, Tensor _3, Tensor _4) -> Tensor",
    "spmm_u_mul_e_sum": "(Tensor _0, Tensor _1, Tensor _2, Tensor _3, Tensor _4, Tensor _5, Tensor _6) -> Tensor",
    "sddmm_u_add_v": "(Tensor _0, Tensor _1, Tensor _2, Tensor _3, Tensor _4, Tensor _5, Tensor _6) -> Tensor",
    "sddmm_u_mul_v": "(Tensor _0, Tensor _1, Tensor _2, Tensor _3, Tensor _4, Tensor _5, Tensor _6) -> Tensor",
    "alltoall": None, "sp_sample_and_shuffle": None,
    "sp_sample_shuffle_src": None, "mp_sample_shuffle": None, "sp_feat_shuffle": None,
    "mp_feat_shuffle_fwd": None, "mp_feat_shuffle_bwd": None,
}


def test_operator_names_and_schemas():
    import torch

    import apt_amd  # noqa: F401  (loads libnpc.so)
    for name, schema in REFERENCE_OPS.items():
        got = torch._C._jit_get_schemas_for_operator(f"npc::{name}")
        assert len(got) == 1, name
        if schema is not None:
            text = re.sub(r" _\d+(?=[,)]|$)", "", str(got[0]).replace(f"npc::{name}", ""))
            want = re.sub(r" _\d+(?=[,)]|$)", "", schema)
            assert text == want, (name, text, want)


def test_peer_operators_raise():
    import torch

    import apt_amd  # noqa: F401
    with pytest.raises(RuntimeError, match="other GPUs"):
        torch.ops.npc.np_sample_and_shuffle(torch.arange(4), 3)
    with pytest.raises(RuntimeError, match="other GPUs"):
        torch.ops.npc.nccl_get_unique_id()


def test_sample_blocks_returns_fresh_tensors_by_default():
    """The registry-owned output ring of sample_blocks is opt-in: by default the operator allocates its
    outputs on every call, like the reference's operators (a result is never overwritten by a later call)."""
    import torch

    import apt_amd
    assert torch.ops.npc.block_buffer_ring() == 0
    apt_amd.ops.set_block_buffer_ring(3)
    assert apt_amd.ops.block_buffer_ring() == 3
    apt_amd.ops.set_block_buffer_ring(0)
    assert torch.ops.npc.block_buffer_ring() == 0
    with pytest.raises(RuntimeError, match="0..64"):
        apt_amd.ops.set_block_buffer_ring(-1)


def test_ctypes_structs_match_the_header(tmp_path):
    """The ctypes mirrors of the ABI's structs have the size and field offsets the C compiler gives them."""
    import subprocess

    from apt_amd import capi
    src = tmp_path / "sizes.c"
    fields = [("apt_graph", capi.CGraph, ["indptr", "adj_pos_map", "num_total_nodes"]),
              ("apt_feat_store", capi.CFeatStore, ["pos_map", "out_dim", "elem_size"]),
              ("apt_batch_slot", capi.CBatchSlot, ["counts", "workspace_bytes", "features", "request_workspace_bytes"]),
              ("apt_epoch_desc", capi.CEpochDesc, ["store", "hop_fanouts", "rank_table_len", "request_pos_map",
                                                   "num_remote_workers", "num_slots", "slots"])]
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "apt_amd.h"', "int main(void) {"]
    for name, _, fs in fields:
        lines.append(f'  printf("%zu\\n", sizeof({name}));')
        lines += [f'  printf("%zu\\n", offsetof({name}, {f}));' for f in fs]
    lines += ['  printf("%zu %d %d %d\\n", sizeof(apt_pending_lookup), APT_MAX_HOPS, APT_MAX_SLOTS, APT_MAX_BUCKETS);',
              "  return 0;", "}"]
    src.write_text("\n".join(lines))
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()
    it = iter(out)
    for name, ct, fs in fields:
        assert int(next(it)) == ctypes.sizeof(ct), name
        for f in fs:
            assert int(next(it)) == getattr(ct, f).offset, (name, f)
    assert [int(x) for x in it] == [512, capi.MAX_HOPS, capi.MAX_SLOTS, 64]


def test_epoch_driver_argument_checks_need_no_gpu():
    from apt_amd import capi
    L = capi.lib()
    h = ctypes.c_void_p()
    d = capi.CEpochDesc()
    assert L.apt_epoch_create(ctypes.byref(d), ctypes.byref(h)) != 0 and b"batch" in L.apt_last_error()
    d.batch, d.num_hops, d.num_slots = 64, 2, 1
    d.hop_fanouts[0], d.hop_fanouts[1] = 5, 5
    assert L.apt_epoch_create(ctypes.byref(d), ctypes.byref(h)) != 0 and b"slot 0" in L.apt_last_error()
    d.num_slots = 17
    assert L.apt_epoch_create(ctypes.byref(d), ctypes.byref(h)) != 0 and b"num_slots" in L.apt_last_error()
    assert not h.value
    # a slot whose sampling buffers are there (never dereferenced by the checks) but whose block buffers are not
    d.num_slots, d.formats = 1, 1
    fan = (ctypes.c_int * 2)(5, 5)
    s = d.slots[0]
    fake = 4096
    p64 = lambda: fake
    s.nodes, s.sizes, s.rank_table, s.workspace = fake, fake, fake, fake
    s.workspace_bytes = L.apt_minibatch_workspace_bytes(64, fan, 2)
    for k in range(2):
        s.neighbors[k], s.relabeled[k] = p64(), p64()
    assert L.apt_epoch_create(ctypes.byref(d), ctypes.byref(h)) != 0 and b"block_edges" in L.apt_last_error()
    s.block_edges = p64()
    assert L.apt_epoch_create(ctypes.byref(d), ctypes.byref(h)) != 0 and b"block buffers of hop 0" in L.apt_last_error()
    for k in range(2):
        b = s.blocks[k]
        b.coo_row, b.coo_col, b.csc_indptr, b.workspace, b.workspace_bytes = p64(), p64(), p64(), fake, 1 << 30
    s.blocks[1].csr_indptr = p64()
    assert L.apt_epoch_create(ctypes.byref(d), ctypes.byref(h)) != 0 and b"all three CSR" in L.apt_last_error()
    s.blocks[1].csr_indices, s.blocks[1].csr_eids, s.blocks[1].workspace_bytes = p64(), p64(), 8
    assert L.apt_epoch_create(ctypes.byref(d), ctypes.byref(h)) != 0 and b"hop 1: block workspace" in L.apt_last_error()
    assert not h.value
    assert L.apt_epoch_next(None, None, None, None) != 0 and L.apt_epoch_release(None, None) != 0
    assert L.apt_epoch_begin(None, None, 0, 0, None) != 0 and L.apt_epoch_end(None) != 0
    assert L.apt_epoch_destroy(None) == 0


def test_bidding_sampler_argument_checks_need_no_gpu():
    """apt_sample_neighbors_bidding rejects what it cannot do before it touches the GPU."""
    from apt_amd import capi
    L = capi.lib()
    g = capi.CGraph()
    table = ctypes.c_void_p(256)                      # never dereferenced by the checks
    assert L.apt_sample_neighbors_bidding(ctypes.byref(g), None, 10, None, 65, 0, 1, 0, None, None, None, 0, table, 100,
                                          ctypes.c_void_p(8), None, ctypes.c_void_p(16), 1 << 20, None) != 0
    assert b"fanout" in L.apt_last_error()
    assert L.apt_sample_neighbors_bidding(ctypes.byref(g), None, 10, None, 5, 0, 1, 0, None, None, None, 0, table, 100,
                                          None, None, ctypes.c_void_p(16), 1 << 20, None) != 0
    assert b"slot_states" in L.apt_last_error()
    assert L.apt_sample_neighbors_bidding(ctypes.byref(g), None, 10, None, 5, 0, 1, 0, None, None, None, 0, None, 100,
                                          ctypes.c_void_p(8), None, ctypes.c_void_p(16), 1 << 20, None) != 0
    assert b"rank table" in L.apt_last_error()
    assert L.apt_sample_neighbors_bidding(ctypes.byref(g), None, 10, None, 5, 0, 1, 0, None, None, None, 0, table, 100,
                                          ctypes.c_void_p(8), None, ctypes.c_void_p(16), 8, None) != 0
    assert b"workspace" in L.apt_last_error()
    # apt_relabel_ranked: a call that takes placed bids over needs neighbours
    assert L.apt_relabel_ranked(ctypes.c_void_p(8), 4, None, None, 0, 0, 2, table, 100, ctypes.c_void_p(8), None,
                                ctypes.c_void_p(8), ctypes.c_void_p(16), None, ctypes.c_void_p(16), 1 << 20, None) != 0
    assert b"neighbours" in L.apt_last_error()
