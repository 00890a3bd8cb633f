"""Drop-in `quik` package: the reference's import surface (quik/__init__.py:1-4 there) served by
the MI355X implementation in quik_amd."""
from quik._C import matmul, symmetric, asymmetric
from quik.version import __version__

__all__ = ['matmul', 'symmetric', 'asymmetric']
