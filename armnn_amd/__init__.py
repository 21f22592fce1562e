"""MI355X-native int8 backend for Arm NN: Python-side helpers.

The product is the C++17 backend under ``armnn_amd/backend`` and the HIP device library under
``armnn_amd/csrc`` (C ABI declared in ``include/armnn_mi355x.h``).  This package only carries what
tests and the benchmark need to drive that C ABI from Python: a ctypes binding, tensor/descriptor
records named after their Arm NN counterparts, seeded synthetic data and the two benchmark networks.
"""
from .tensor import DataType, TensorInfo, QTensor  # noqa: F401
