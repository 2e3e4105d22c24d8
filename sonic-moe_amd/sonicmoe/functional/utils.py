"""`enable_quack_gemm` exists in the reference to switch to a second GEMM implementation
(sonicmoe/functional/utils.py:9-25).  This package has exactly one GEMM path, so the context manager is accepted for
source compatibility and changes nothing."""

from contextlib import contextmanager


@contextmanager
def enable_quack_gemm(enable: bool = True):
    yield


def is_using_quack_gemm() -> bool:
    return False
