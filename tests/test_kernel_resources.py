"""Resource budgets of the hot kernels, read from the compiler's own remarks
(-Rpass-analysis=kernel-resource-usage while cross-compiling for gfx950; no GPU needed).

A launch of the gather is capped at the 2048 workgroups the CUs hold at once (8 waves per SIMD), which they
only do while the kernel allocates at most 64 VGPRs per lane and no scratch; registers are allocated in
granules of 8, and the shipped row loop (16-byte vectors, two rows in flight, the ids of the next iteration
fetched at the end of the one before) uses 44.  Nothing in a functional test notices when an edit or a compiler
takes a kernel over such a limit or makes it spill, so the budgets are asserted here from the compiler's own
figures.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "apt_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

pytestmark = pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")


def _build_flags():
    """The flags the library is built with (apt_amd/build.py, loaded by path: importing the package needs
    the built libraries)."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("_apt_amd_build", os.path.join(ROOT, "apt_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return list(mod.FLAGS)


def _resources(source, tmp_path):
    """-> {demangled kernel name: {remark field: int}} for every kernel of one source file."""
    cmd = [HIPCC, *_build_flags(), "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage", "-c",
           os.path.join(CSRC, source), "-o", str(tmp_path / (source + ".o"))]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-3000:]
    kernels, cur = {}, None
    for line in r.stderr.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            cur = kernels.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+) \[-Rpass", line)
        if m and cur is not None:
            cur[m.group(1).strip()] = int(m.group(2))
    assert kernels, "the compiler printed no resource remarks:\n" + r.stderr[-2000:]
    names = list(kernels)
    dem = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True, check=True).stdout.splitlines()
    return {d: kernels[n] for d, n in zip(dem, names)}


def _one(res, prefix):
    hits = [k for k in res if k.startswith(prefix)]
    assert len(hits) == 1, (prefix, sorted(res))
    return res[hits[0]]


def test_gather_kernels_keep_full_occupancy_and_do_not_spill(tmp_path):
    res = _resources("gather.hip", tmp_path)
    # the shipped shapes: 16-byte vectors, two rows per lane group in flight, 16 lanes per row (256-byte rows),
    # 32 (512-byte rows) and 8 (128-byte rows); the variant that carries the relabel's last pass
    for name in ("void apt::gather_kernel<16, 16, 2>(", "void apt::gather_kernel<16, 32, 2>(",
                 "void apt::gather_kernel<16, 8, 2>(", "void apt::gather_with_lookup_kernel<16>(",
                 "void apt::gather_with_lookup_kernel<32>("):
        k = _one(res, name)
        assert k["VGPRs"] <= 48, (name, k)                       # measured at 44; 8 waves per SIMD need <= 64
        assert k["Occupancy"] >= 8, (name, k)                    # 8 waves per SIMD: 2048 co-resident workgroups
        assert k["ScratchSize"] == 0 and k["VGPRs Spill"] == 0 and k["SGPRs Spill"] == 0, (name, k)
        assert k["LDS Size"] == 0, (name, k)
    # no gather variant may spill, whatever its shape
    for name, k in res.items():
        if "gather" in name:
            assert k["ScratchSize"] == 0 and k["VGPRs Spill"] == 0, (name, k)


def test_sampling_kernels_do_not_spill(tmp_path):
    res = _resources("sample.hip", tmp_path)
    hop3 = _one(res, "void apt::sample_kernel<16, false, 1>(")    # the last hop of fan_out 15,10,5
    # (scalar registers that do not fit are parked in lanes of a vector register, not in memory: the kernel's
    # argument block alone is 50 of the 102 it may use, so a few dozen such moves are expected and harmless)
    assert hop3["ScratchSize"] == 0 and hop3["VGPRs Spill"] == 0, hop3
    assert hop3["VGPRs"] <= 64, hop3                              # 8 waves per SIMD by registers (LDS allows 7)
    assert hop3["Occupancy"] >= 4, hop3                           # 512-thread workgroups: at least two per CU
    for name, k in res.items():
        if "sample_kernel" in name:
            assert k["ScratchSize"] == 0 and k["VGPRs Spill"] == 0, (name, k)
            assert k["LDS Size"] <= 64 * 1024, (name, k)


def test_relabel_kernels_fit_lds_and_do_not_spill(tmp_path):
    res = _resources("relabel.hip", tmp_path)
    lds = _one(res, "apt::relabel_lds_kernel(")
    assert lds["LDS Size"] <= 160 * 1024, lds                     # one workgroup holds keys and table in LDS
    assert lds["LDS Size"] >= 128 * 1024, lds                     # and it really is the LDS-resident design
    for name, k in res.items():
        assert k["ScratchSize"] == 0 and k["VGPRs Spill"] == 0, (name, k)


def test_minibatch_kernels_do_not_spill(tmp_path):
    res = _resources("minibatch.hip", tmp_path)
    assert any("mb_place_kernel" in n for n in res) and any("mb_count_kernel" in n for n in res)
    for name, k in res.items():
        assert k["ScratchSize"] == 0 and k["VGPRs Spill"] == 0, (name, k)
