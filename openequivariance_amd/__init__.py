"""MI355X-native equivariant tensor products with the OpenEquivariance API.

``import openequivariance_amd as oeq`` gives ``oeq.TPProblem``, ``oeq.Irreps``,
``oeq.TensorProduct`` and ``oeq.TensorProductConv`` with the reference's
signatures (openequivariance/openequivariance/__init__.py:9-116). Set
``OEQ_NOTORCH=1`` to import only the numpy-level specification classes.
"""

import os

import numpy as np

from .core.spec import Instruction, Irrep, Irreps, TPProblem, _MulIr

__version__ = "0.1.0"

if os.environ.get("OEQ_NOTORCH") != "1":
    import torch

    from ._torch.tensor_product import TensorProduct
    from ._torch.tensor_product_conv import TensorProductConv
    from ._torch.utils import torch_to_oeq_dtype, transpose_irreps

    from .core.problems import ChannelwiseTPP, FullyConnectedTPProblem, SingleInstruction

    torch.serialization.add_safe_globals(
        [TensorProduct, TensorProductConv, TPProblem, Irrep, Irreps, _MulIr, Instruction, np.float32, np.float64,
         ChannelwiseTPP, FullyConnectedTPProblem, SingleInstruction]
    )


def torch_ext_so_path():
    """Path of the C-ABI shared library behind the torch ops."""
    from . import runtime
    return str(runtime.lib_path())


__all__ = ["TPProblem", "Irrep", "Irreps", "Instruction", "TensorProduct", "TensorProductConv",
           "torch_to_oeq_dtype", "transpose_irreps", "torch_ext_so_path"]
