"""Builds and binds the host lane-simulator flavour of the kernel library (test infrastructure).

The simulator runs the unchanged kernel sources on the CPU, so these tests exercise the kernels'
index arithmetic, masking and numerics -- and the C entry points and Python marshalling -- without a
GPU.  The shipped package never loads this library.
"""
import os
import subprocess

from flagattention_amd import _lib

HERE = os.path.dirname(os.path.abspath(__file__))
PATH = os.path.join(HERE, "libflagattn_sim.so")

_bound = None


def get():
    global _bound
    if _bound is None:
        subprocess.run(["make", "-s", "-j8", "-C", HERE], check=True)
        _bound = _lib.bind(PATH)
    return _bound
