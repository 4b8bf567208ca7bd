"""ascq: Python binding of libascq, the MI355X implementation of the asc-devkit quantization operators.

`ascq._abi` is the raw C ABI (enums, descriptor structs, loader); `ascq.ops` mirrors the reference's operator
interface (AscendQuant, AscendDequant, AscendAntiQuant, Matmul with SetQuantScalar/SetQuantVector, grouped matmul,
W4A16) on torch device tensors.  torch is used for device memory and streams only.
"""
from . import _abi  # noqa: F401

__all__ = ["_abi", "ops"]


def __getattr__(name):
    if name == "ops":
        import importlib
        return importlib.import_module(".ops", __name__)
    raise AttributeError(name)
