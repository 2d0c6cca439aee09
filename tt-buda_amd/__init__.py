"""MI355X-native block-floating-point data-format path of TT-Buda.

Layers, bottom up:
  libttbfp.so   HIP kernels for gfx950 + the C ABI of include/ttbfp.h      (csrc/device)
  _C            C++ host layer behind pybind11: DataFormat, descriptors,
                queues in HBM and the tt::backend entry points             (csrc/host)
  capi          ctypes view of the C ABI on torch device tensors
  tensor        torch <-> descriptor glue (dtype maps, padding, narrowing)
  backend       push / read / pop loops over the queues
  op            matmul / GELU / FFN with Bfp8_b weights
  tti           tensor entries of a saved device image (.bin / .tbin payloads and their JSON)
"""
import os as _os

_pkg = __path__[0]  # noqa: F821 (also right when imported through the tt_buda_amd alias)
if not _os.path.exists(_os.path.join(_pkg, "libttbfp.so")):
    raise ImportError(
        "tt_buda_amd: libttbfp.so has not been built; run `python -c 'import __graft_entry__ as g; g.build()'`")

# torch first: it bundles its own HIP runtime (same soname as the system one), and a process must
# not end up with torch running on a runtime that libttbfp.so pulled in before it.
import torch as _torch  # noqa: E402,F401

from . import _C  # noqa: E402,F401
from . import backend, capi, op, tensor, tti  # noqa: E402,F401
from ._C import DataFormat, MathFidelity  # noqa: E402,F401
from .capi import DataFormatCode  # noqa: E402,F401
