"""Editable install of the MI355X page-copy path: `pip install -e bi-kv_amd` (or `python setup.py develop`).

Takes the place of Bi-KV/SharedMemory/CUDA_Shared/setup.py:4-22, which builds the reference's `ipc_service`
pybind module from ipc_service.cpp + copy_kernel.cu with nvcc. Here the native part is a plain C-ABI shared
library built by csrc/Makefile (hipcc, gfx950; no torch headers, no pybind) into lib/, and `ipc_service` /
`bikv_pagecopy` are Python packages that load it with ctypes from that in-tree location — so the install must
be an editable one (the packages look for ../lib/libbikv_pagecopy.so next to themselves).
"""
import os
import subprocess

from setuptools import Command, setup
from setuptools.command.build_py import build_py
from setuptools.command.develop import develop

HERE = os.path.dirname(os.path.abspath(__file__))


def build_native():
    subprocess.check_call(["make", "-C", os.path.join(HERE, "csrc"), "-j4"])


class BuildNative(Command):
    description = "build lib/libbikv_pagecopy.so with hipcc for gfx950"
    user_options = []

    def initialize_options(self):
        pass

    def finalize_options(self):
        pass

    def run(self):
        build_native()


class BuildPy(build_py):
    def run(self):
        build_native()
        super().run()


class Develop(develop):
    def run(self):
        build_native()
        super().run()


setup(
    name="bikv_pagecopy",
    version="1.0",
    description="MI355X-native KV page gather/scatter for Bi-KV behind its ipc_service operator API",
    packages=["bikv_pagecopy", "ipc_service"],
    package_dir={"": "."},
    cmdclass={"build_native": BuildNative, "build_py": BuildPy, "develop": Develop},
)
