import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "llumnix-kv_amd"), os.path.join(ROOT, "tests"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_sessionstart(session):
    """Tests load what is built; only when nothing is built yet (a fresh checkout) is the
    library compiled first (hipcc cross-compiles without a GPU)."""
    import shutil
    import subprocess
    so = os.path.join(ROOT, "llumnix-kv_amd", "libkvt_hip.so")
    have_hipcc = shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")
    if not os.path.exists(so) and have_hipcc:
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "llumnix-kv_amd"), "-j8"])
