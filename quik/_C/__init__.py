"""`quik._C`: in the reference a pybind11 extension with three submodules (src/binding.cpp:7-11);
here the same three namespaces, backed by libquik_hip.so through quik_amd."""
from quik_amd import asymmetric, matmul, symmetric

__all__ = ["matmul", "symmetric", "asymmetric"]
