"""MI355X-native butterfly matrix multiply.

Importing the package loads the native libraries built by ``python -m butterfly_amd.build``
and registers the ``torch.ops.torch_butterfly.*`` operators.  There is no fallback: if the
libraries are missing the import fails.
"""
import os

import torch

__version__ = "0.1.0"

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))


def _load_native():
    # Same discovery rule as the reference initialiser (torch_butterfly/__init__.py:8-11):
    # two operator libraries, found by bare name next to this file.
    for name in ("_version", "_butterfly"):
        path = os.path.join(_PKG_DIR, name + ".so")
        if not os.path.isfile(path):
            raise ImportError(
                f"{path} is missing: build the native libraries with `python -m butterfly_amd.build`")
        torch.ops.load_library(path)


_load_native()

from .multiply import butterfly_multiply  # noqa: E402
from .multiply_base4 import butterfly_multiply_base4  # noqa: E402
from .butterfly import Butterfly, ButterflyBmm, ButterflyUnitary  # noqa: E402
from .butterfly_base4 import ButterflyBase4  # noqa: E402
from .graphed import GraphedStep  # noqa: E402
from . import combine, complex_utils, diagonal, kops, legacy, legacy_permutation, multiply, multiply_base4, permutation, special  # noqa: E402,F401

__all__ = [
    "Butterfly",
    "ButterflyBase4",
    "ButterflyBmm",
    "ButterflyUnitary",
    "GraphedStep",
    "butterfly_multiply",
    "butterfly_multiply_base4",
    "__version__",
]
