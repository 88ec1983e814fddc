"""The installable form of the package (the counterpart of the reference's
setup.py:16-40 and README.md:31-39): a wheel is built offline, unpacked into
an empty directory, and imported from there by a fresh interpreter that sees
nothing of the source tree.  Both shared objects must travel, the binding
must find the kernel library through its $ORIGIN rpath, and the package
version must be the distribution's.  No GPU is needed (nothing is launched)."""
import glob
import os
import subprocess
import sys
import zipfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "warp-ctct_amd")

PROBE = r"""
import os, sys
import warp_ctct
from warp_ctct import _C
from importlib.metadata import version
maps = open("/proc/self/maps").read()
libs = sorted({line.split()[-1] for line in maps.splitlines() if "libwarpctct_hip.so" in line})
print("PKG", os.path.dirname(os.path.abspath(warp_ctct.__file__)))
print("BINDING", os.path.abspath(_C.__file__))
print("KERNELS", ";".join(libs))
print("VERSION", warp_ctct.__version__, version("warp_ctct"), _C.library_version())
print("API", ",".join(sorted(warp_ctct.__all__)))
"""


def test_wheel_builds_unpacks_and_imports_outside_the_source_tree(tmp_path):
    tmp = str(tmp_path)
    env = dict(os.environ, PYTORCH_ROCM_ARCH="gfx950")
    cmd = [sys.executable, "setup.py", "-q", "egg_info", "--egg-base", tmp,
           "build", "--build-base", os.path.join(tmp, "build"),
           "bdist_wheel", "--dist-dir", os.path.join(tmp, "dist")]
    done = subprocess.run(cmd, cwd=PKG, env=env, capture_output=True, text=True, timeout=900)
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-4000:]
    wheels = glob.glob(os.path.join(tmp, "dist", "warp_ctct-*.whl"))
    assert len(wheels) == 1, wheels
    with zipfile.ZipFile(wheels[0]) as z:
        names = z.namelist()
        unpacked = os.path.join(tmp, "unpacked")
        z.extractall(unpacked)
    assert "warp_ctct/__init__.py" in names
    assert "warp_ctct/libwarpctct_hip.so" in names, names
    assert any(n.startswith("warp_ctct/_C") and n.endswith(".so") for n in names), names
    meta = [n for n in names if n.endswith(".dist-info/METADATA")]
    assert len(meta) == 1
    text = open(os.path.join(unpacked, meta[0])).read()
    dist_version = [l.split(":", 1)[1].strip() for l in text.splitlines() if l.startswith("Version:")][0]
    # zipfile drops the executable bit; shared objects do not need it to be loaded
    clean = {k: v for k, v in os.environ.items() if k not in ("PYTHONPATH", "LD_LIBRARY_PATH")}
    clean["PYTHONPATH"] = unpacked
    out = subprocess.run([sys.executable, "-c", PROBE], cwd=unpacked, env=clean, capture_output=True,
                         text=True, timeout=600)
    assert out.returncode == 0, out.stdout + out.stderr[-4000:]
    fields = dict(line.split(" ", 1) for line in out.stdout.strip().splitlines())
    real = os.path.realpath(unpacked)
    assert os.path.realpath(fields["PKG"]) == os.path.join(real, "warp_ctct")
    assert os.path.realpath(fields["BINDING"]).startswith(os.path.join(real, "warp_ctct", "_C"))
    kernels = fields["KERNELS"].split(";")
    assert len(kernels) == 1, kernels
    assert os.path.realpath(kernels[0]) == os.path.join(real, "warp_ctct", "libwarpctct_hip.so")
    pkg_version, meta_version, lib_version = fields["VERSION"].split()
    # the distribution and the package carry the reference distribution's version
    # (setup.py:18 of the reference); the kernel library's ABI version is its own
    assert pkg_version == meta_version == dist_version == "0.3.0"
    assert lib_version.count(".") == 2
    # exactly the reference's export list (warp_ctct/__init__.py:17 of the reference)
    assert fields["API"] == "ctct_loss,ctct_simple_loss"
