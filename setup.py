"""`pip install .` for the gfx950 selective_nd_scan: same distribution name as the reference
(kernels/selective_nd_scan/setup.py:118, `selective_nd_scan`) and the same importable extension name
(`selective_nd_scan_cuda_oflex`, setup.py:80), built by hipcc for gfx950 only.  Unlike the reference's
setup.py (:24-27,48) no GPU is needed at build time."""
import importlib.util
import os
import shutil

from setuptools import setup
from setuptools.command.build_py import build_py

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "official-cross-scan_amd")


def _build_native():
    spec = importlib.util.spec_from_file_location("snd_build", os.path.join(PKG, "build.py"))
    b = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(b)
    return [b.build_capi(), b.build_torch_ext()]


class BuildWithNative(build_py):
    """Compile libsnd_scan.so and the PyTorch extension in-tree, then ship them next to the modules."""

    def run(self):
        built = _build_native()
        super().run()
        for path in built:
            shutil.copy2(path, os.path.join(self.build_lib, os.path.basename(path)))
        os.makedirs(os.path.join(self.build_lib, "include"), exist_ok=True)


setup(
    name="selective_nd_scan",
    version="2.0.0",
    description="2D-CrossScan selective scan (forward + backward) for AMD MI355X / gfx950",
    package_dir={"": "official-cross-scan_amd"},
    packages=["selective_nd_scan"],
    py_modules=["selective_nd_scan_cuda_oflex"],
    cmdclass={"build_py": BuildWithNative},
    python_requires=">=3.9",
)
