"""`pip install .` (the reference's install route, README.md:11 / setup.py:1-17): the tree
installs into an empty directory as module `quadmul` + package `quadmul_amd`, and both import
from there -- the extension finding libqm_hip.so through its $ORIGIN rpath -- from a process
that cannot see the repository.  The libraries already built in the tree are reused
(QM_REUSE_BUILD=1): compiling is `python -m quadmul_amd.build`'s job and is checked by the
build step; this test is about the packaging."""
import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_pip_install_into_a_prefix_and_import_from_outside(tmp_path):
    target = tmp_path / "site"
    leftovers = [p for p in (os.path.join(ROOT, "build"), os.path.join(ROOT, "quadmul.egg-info")) if not os.path.exists(p)]
    env = dict(os.environ, QM_REUSE_BUILD="1", PIP_DISABLE_PIP_VERSION_CHECK="1")
    r = subprocess.run([sys.executable, "-m", "pip", "install", "--no-build-isolation", "--no-deps", "--no-index", "--target", str(target), ROOT],
                       capture_output=True, text=True, env=env, timeout=600)
    for p in leftovers:   # what pip's in-tree build leaves behind
        shutil.rmtree(p, ignore_errors=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    names = os.listdir(target)
    assert any(n.startswith("quadmul.") and n.endswith(".so") for n in names), names
    assert os.path.exists(target / "quadmul_amd" / "lib" / "libqm_hip.so")
    assert not os.path.exists(target / "quadmul_amd" / "lib" / "libqm_probe.so")   # bench.py's instruments stay in the tree
    code = ("import sys, os; assert not any(os.path.abspath(p or '.') == %r for p in sys.path); "
            "import quadmul, quadmul_amd; "
            "assert quadmul.__file__.startswith(%r) and quadmul_amd.__file__.startswith(%r); "
            "assert quadmul.num_configs() == quadmul_amd.num_configs() > 10; "
            "assert 'Int4xInt4' in quadmul.gemm.__doc__; print(quadmul.version())") % (ROOT, str(target), str(target))
    env2 = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    env2["PYTHONPATH"] = str(target)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=str(tmp_path), env=env2, timeout=300)
    assert r.returncode == 0 and "quadmul-amd" in r.stdout, r.stdout[-2000:] + r.stderr[-3000:]
