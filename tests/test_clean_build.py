"""The build entry point must work on a tree that holds sources only (what `git archive` gives):
no prebuilt library may be needed to produce the libraries."""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILT = (".so", ".o", ".a", ".hsaco", ".co", ".pyc", ".tmp")


def _source_files():
    """What a commit of the tree holds: tracked files plus untracked ones that .gitignore does not list."""
    r = subprocess.run(["git", "ls-files", "-co", "--exclude-standard"], cwd=ROOT, capture_output=True, text=True)
    if r.returncode != 0:
        pytest.skip("not a git checkout: " + r.stderr.strip()[:200])
    return [f for f in r.stdout.splitlines() if f and not f.endswith(BUILT) and os.path.isfile(os.path.join(ROOT, f))]


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_build_from_sources_only(tmp_path):
    tree = tmp_path / "tree"
    for f in _source_files():
        dst = tree / f
        dst.parent.mkdir(parents=True, exist_ok=True)
        shutil.copy2(os.path.join(ROOT, f), dst)
    assert not list(tree.rglob("*.so"))
    code = ("import __graft_entry__ as g; g.build(); import apt_amd, os; "
            "assert os.path.dirname(apt_amd.__file__).startswith(os.getcwd()), apt_amd.__file__; print('built')")
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    r = subprocess.run([sys.executable, "-c", code], cwd=tree, env=env, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    assert "built" in r.stdout
    for so in ("apt_amd/libapt_hip.so", "apt_amd/libapt_bench.so", "apt_amd/libnpc.so", "oracle/liborc.so"):
        assert (tree / so).exists(), so
