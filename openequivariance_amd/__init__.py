"""MI355X-native Clebsch-Gordan tensor products and fused equivariant graph convolution.

Public surface (same names as the reference's ``openequivariance`` package,
reference: openequivariance/__init__.py:4-10):

    TPProblem, Irreps, TensorProduct, TensorProductConv, LoopUnrollTP, LoopUnrollConv

Importing the package does not build or load anything; the C-ABI runtime library is loaded
on first use and must have been built with ``python -m openequivariance_amd.build_ext``.
"""
from .irreps import Irrep, Irreps
from .problem import (ChannelwiseTPP, FullyConnectedTPProblem, Instruction, SingleInstruction, TPProblem)
from .wigner import wigner_3j
from .tensor_product import LoopUnrollTP, TensorProduct
from .conv import (CoordGraph, LoopUnrollConv, LoopUnrollConvAtomic, LoopUnrollConvDeterministic,
                   LoopUnrollConvScatterSum, TensorProductConv, sort_by_receiver)

__all__ = ["Irrep", "Irreps", "TPProblem", "Instruction", "ChannelwiseTPP", "FullyConnectedTPProblem",
           "SingleInstruction", "wigner_3j", "TensorProduct", "TensorProductConv", "LoopUnrollTP",
           "LoopUnrollConv", "LoopUnrollConvAtomic", "LoopUnrollConvDeterministic", "LoopUnrollConvScatterSum",
           "CoordGraph", "sort_by_receiver"]
