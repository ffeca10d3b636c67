"""The Node-API shim: the reference's JavaScript-side call pattern against the
HIP engine, run under the Node binary of this image."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ADDON = os.path.join(ROOT, "framework_amd", "lib", "mni_rocm.node")


@pytest.mark.gpu
def test_javascript_callers_through_the_addon():
    node = shutil.which("node")
    if node is None:
        pytest.skip("no node binary on this machine")
    if not os.path.exists(ADDON):
        pytest.skip("Node addon not built (node_api.h missing at build time)")
    p = subprocess.run([node, os.path.join(ROOT, "tests", "js", "matmul_path.js")], capture_output=True, text=True, timeout=120)
    print(p.stdout, p.stderr)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "0 failed" in p.stdout


def test_addon_source_exports_every_engine_function():
    # every mni_* engine function the header declares is reachable from the shim
    import re
    header = open(os.path.join(ROOT, "include", "mni_rocm.h")).read()
    shim = open(os.path.join(ROOT, "framework_amd", "csrc", "napi_shim.cpp")).read()
    engine = sorted(set(re.findall(r"\b(mni_(?!rocm_)[a-z0-9_]+)\s*\(", header)))
    missing = [f for f in engine if f not in shim and f != "mni_dev_ptr"]
    assert not missing, missing
