"""Packaging of fp8_gmm_amd: ``pip install -e .`` (or ``pip install .``) builds ``libfp8gmm_hip.so`` with the
Makefile under ``fp8_gmm_amd/csrc`` (hipcc, gfx950) and ships it inside the package, next to ``_lib.py`` that loads
it.  Takes the place of the reference's ``setup.py`` (a torch CUDAExtension named ``fp8_gmm_backend``, setup.py:26-44)
and ``reinstall.sh``: the library here is a plain C-ABI shared object, not a Python extension module, so no torch
headers are involved in building it."""
import os
import subprocess

from setuptools import Command, find_packages, setup
from setuptools.command.build_py import build_py
from setuptools.command.develop import develop

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "fp8_gmm_amd", "csrc")


def make_library():
    jobs = os.environ.get("MAX_JOBS", str(min(16, os.cpu_count() or 1)))
    subprocess.check_call(["make", "-C", CSRC, f"-j{jobs}"])


class BuildHip(Command):
    description = "build libfp8gmm_hip.so (hipcc, --offload-arch=gfx950)"
    user_options = []

    def initialize_options(self):
        pass

    def finalize_options(self):
        pass

    def run(self):
        make_library()


class BuildPy(build_py):
    def run(self):
        self.run_command("build_hip")
        super().run()


class Develop(develop):
    def run(self):
        self.run_command("build_hip")
        super().run()


setup(
    name="fp8_gmm_amd",
    version="0.3.0",
    description="FP8 grouped GEMM modules for MoE expert layers on MI355X (gfx950): hand-written HIP behind a C ABI",
    packages=find_packages(include=["fp8_gmm_amd", "fp8_gmm_amd.*"]),
    package_data={"fp8_gmm_amd": ["libfp8gmm_hip.so"]},
    python_requires=">=3.10",
    install_requires=["numpy"],   # torch is expected to be the ROCm build already present
    cmdclass={"build_hip": BuildHip, "build_py": BuildPy, "develop": Develop},
)
