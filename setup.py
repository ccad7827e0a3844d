"""`pip install .` for the MI355X packed-int4 GEMM: installs the drop-in extension module
`quadmul` (same module name as the reference's setup.py:8-11) and the package `quadmul_amd`
with its gfx950 library.

    pip install --no-build-isolation .

The build step is `quadmul_amd.build`: hipcc compiles the HIP kernels for gfx950 into
quadmul_amd/lib/libqm_hip.so, the host compiler compiles the PyTorch extension against
torch's headers (no CUDAExtension and none of torch's source translation: nothing here is
CUDA).  `--no-build-isolation` because the extension is built against the torch that is
installed.  QM_REUSE_BUILD=1 installs the libraries already built in the tree instead of
compiling again.
"""
import os
import shutil
import sys

from setuptools import Extension, setup
from setuptools.command.build_ext import build_ext

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


class BuildNative(build_ext):
    """Runs the in-tree build recipe and copies what it made to where setuptools installs from."""

    def run(self):
        from quadmul_amd import build as qbuild

        # (the measurement probes of bench.py, libqm_probe.so, stay in the tree: a user of the
        # library has no use for them)
        libs = [qbuild.LIB_PATH]
        reuse = os.environ.get("QM_REUSE_BUILD") == "1" and all(os.path.exists(p) for p in libs + [qbuild.ext_path()])
        if not reuse:
            qbuild.build_lib(jobs=int(os.environ.get("MAX_JOBS", "8")))
            qbuild.build_ext()
        # the extension module: looks for libqm_hip.so in quadmul_amd/lib beside it ($ORIGIN rpath)
        dst = self.get_ext_fullpath("quadmul")
        os.makedirs(os.path.dirname(dst), exist_ok=True)
        if os.path.abspath(dst) != os.path.abspath(qbuild.ext_path()):
            shutil.copy2(qbuild.ext_path(), dst)
        if not self.inplace:
            libdir = os.path.join(self.build_lib, "quadmul_amd", "lib")
            os.makedirs(libdir, exist_ok=True)
            for p in libs:
                shutil.copy2(p, libdir)

    def get_outputs(self):
        outs = [self.get_ext_fullpath("quadmul")]
        if not self.inplace:
            outs += [os.path.join(self.build_lib, "quadmul_amd", "lib", "libqm_hip.so")]
        return outs


setup(
    name="quadmul",
    version="0.3",
    description="Packed int4 x int4 -> int32 GEMM for AMD MI355X (gfx950): drop-in for quadmul.gemm",
    packages=["quadmul_amd"],
    package_data={"quadmul_amd": ["csrc/*", "lib/libqm_hip.so"]},
    ext_modules=[Extension("quadmul", sources=[])],   # built by quadmul_amd.build, not by setuptools
    cmdclass={"build_ext": BuildNative},
    python_requires=">=3.9",
    zip_safe=False,
)
