"""Install the MI355X FBW / best-path package with `pip install --no-build-isolation .` in this directory
(PyTorch-ROCm and hipcc must be there already; nothing is downloaded).

Takes the place of the reference's setup.py (setup.py:25-64, four CUDAExtensions built by torch's
BuildExtension): the native parts -- libi6fbw.so (HIP kernels + C ABI, hipcc for gfx950) and the two
PyTorch bindings that link it -- are built by i6_native_ops_amd/build.py, here into the build tree, so
that the installed package carries them next to its Python modules exactly as the in-tree build does.
"""
import importlib.util
import os

from setuptools import Distribution, find_packages, setup
from setuptools.command.build_py import build_py

TOP = os.path.dirname(os.path.abspath(__file__))


def _native_build():
    # loaded by path: the package itself cannot be imported before its extensions exist
    spec = importlib.util.spec_from_file_location("_i6_native_build", os.path.join(TOP, "i6_native_ops_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


class BuildWithNative(build_py):
    def run(self):
        super().run()
        try:
            import torch  # noqa: F401
        except ModuleNotFoundError as exc:
            raise RuntimeError("Please install PyTorch (ROCm build) before installing this package.") from exc
        _native_build().build_all(os.path.join(self.build_lib, "i6_native_ops_amd"))


class BinaryDistribution(Distribution):
    def has_ext_modules(self):      # the wheel holds machine code: tag it for this platform and interpreter
        return True


def _version():
    scope = {}
    exec(open(os.path.join(TOP, "i6_native_ops_amd", "_version.py")).read(), scope)
    return scope["__version__"]


setup(
    name="i6_native_ops_amd",
    version=_version(),
    description="Full-sum forward-backward (FBW) loss and best-path alignment of rwth-i6/i6_native_ops for AMD MI355X (gfx950)",
    packages=find_packages(include=["i6_native_ops_amd", "i6_native_ops_amd.*"]),
    package_data={"i6_native_ops_amd": ["csrc/*.hip", "csrc/*.inc", "csrc/*.cpp", "csrc/*.h", "fbw/*.so", "fast_viterbi/*.so"]},
    cmdclass={"build_py": BuildWithNative},
    distclass=BinaryDistribution,
    python_requires=">=3.9",
)
