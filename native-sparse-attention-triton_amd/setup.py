"""Packaging of native_sparse_attention for MI355X (gfx950): `pip install -e .` (or `python setup.py develop`)
compiles csrc/*.hip with hipcc into native_sparse_attention/lib/libnsa_hip.so (build.py) and installs the
package under the import name the reference uses, so `from native_sparse_attention.ops import ...` keeps working."""
import os
import sys

from setuptools import find_packages, setup
from setuptools.command.build_py import build_py

HERE = os.path.dirname(os.path.abspath(__file__))


class BuildWithHip(build_py):
    def run(self):
        sys.path.insert(0, HERE)
        import build as nsa_build  # build.py next to this file

        nsa_build.build(force=False)
        super().run()


setup(
    name="native-sparse-attention-mi355x",
    version="0.1.0",
    description="Native Sparse Attention operators as hand-written HIP kernels for AMD MI355X (gfx950)",
    packages=find_packages(where=HERE, include=["native_sparse_attention", "native_sparse_attention.*"]),
    package_dir={"": "."},
    package_data={"native_sparse_attention": ["lib/*.so"]},
    install_requires=["torch>=2.1.0"],
    python_requires=">=3.9",
    cmdclass={"build_py": BuildWithHip},
)
