"""Build of the MI355X CTC-Transducer loss.

    python setup.py build_ext --inplace          # in-tree, what the tests and bench.py load
    pip install --no-build-isolation .           # or as an installed package (wheel: bdist_wheel)

1. `make` compiles the HIP kernels + C ABI into warp_ctct/libwarpctct_hip.so
   (hipcc, --offload-arch=gfx950).
2. The torch binding warp_ctct/_C*.so is host-only C++ (no device code); it is
   linked against that library with an $ORIGIN rpath.
The counterpart of the reference's setup.py:16-40 (CUDAExtension "warp_ctct._C").
"""
import os
import subprocess

from setuptools import setup
from torch.utils.cpp_extension import BuildExtension, CppExtension

HERE = os.path.dirname(os.path.abspath(__file__))

# The distribution carries the version of the reference distribution whose API
# it implements (setup.py:18 of the reference: 0.3.0), so that code gating on
# warp_ctct.__version__ behaves the same; the kernel library's own ABI version
# (warpctct_version()) is separate.
with open(os.path.join(HERE, "warp_ctct", "_version.py")) as fh:
    VERSION = fh.read().split('"')[1]
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


class BuildWithHip(BuildExtension):
    def run(self):
        subprocess.check_call(["make", "-C", HERE, "-j4"])
        super().run()


ext = CppExtension(
    name="warp_ctct._C",
    sources=["csrc/binding.cpp"],
    include_dirs=[os.path.join(HERE, "..", "include"), os.path.join(ROCM, "include")],
    define_macros=[("__HIP_PLATFORM_AMD__", "1"), ("USE_ROCM", "1")],
    extra_compile_args=["-O2", "-std=c++17"],
    library_dirs=[os.path.join(HERE, "warp_ctct"), os.path.join(ROCM, "lib")],
    libraries=["warpctct_hip", "c10_hip", "torch_hip", "amdhip64"],
    extra_link_args=["-Wl,-rpath,$ORIGIN"],
)

setup(
    name="warp_ctct",
    version=VERSION,
    description="MI355X (gfx950) CTC-Transducer loss with the warp_ctct API",
    packages=["warp_ctct"],
    # the HIP kernels + C ABI travel with the package, next to the binding that
    # finds them through its $ORIGIN rpath
    package_data={"warp_ctct": ["libwarpctct_hip.so"]},
    python_requires=">=3.8",
    install_requires=["torch>=2.0"],
    ext_modules=[ext],
    cmdclass={"build_ext": BuildWithHip.with_options(use_ninja=False)},
)
