"""The build entry point must work on a tree that holds sources only (what `git archive` gives):
no prebuilt library may be needed to produce the libraries."""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILT = (".so", ".o", ".a", ".hsaco", ".co", ".pyc", ".tmp")
SKIP_DIRS = {".git", "gpurun_out", "_work", "__pycache__", ".pytest_cache", ".hypothesis", "_ref", "profiles"}


def _ignore(_dir, names):
    return [n for n in names if n in SKIP_DIRS or n.endswith(BUILT)]


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_build_from_sources_only(tmp_path):
    tree = tmp_path / "tree"
    shutil.copytree(ROOT, tree, ignore=_ignore)
    assert not list(tree.rglob("*.so"))
    code = ("import __graft_entry__ as g; g.build(); import apt_amd, os; "
            "assert os.path.dirname(apt_amd.__file__).startswith(os.getcwd()), apt_amd.__file__; print('built')")
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    r = subprocess.run([sys.executable, "-c", code], cwd=tree, env=env, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    assert "built" in r.stdout
    for so in ("apt_amd/libapt_hip.so", "apt_amd/libnpc.so", "oracle/liborc.so"):
        assert (tree / so).exists(), so
