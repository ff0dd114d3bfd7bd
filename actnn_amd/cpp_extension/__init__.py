"""Operator surface of the reference's four extension modules
(actnn/setup.py:6-21: actnn.cpp_extension.{calc_precision,minimax,backward_func,quantization}),
implemented over the C ABI in include/actnn_hip.h."""
from . import minimax, quantization, calc_precision, backward_func  # noqa: F401
