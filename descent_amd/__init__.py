"""descent_amd: MI355X (gfx950) execution backend for the descent graph library.

`csrc/` holds the HIP/C++ library behind the C ABI in include/descent_hip.h;
the Python modules mirror the reference's host-side interface (Environment,
Scope/Array/DualArray, Module, optimisers) and drive that ABI through ctypes.
"""
from .array import Array, DualArray, Parameter, Scope
from .environment import Environment
from .graph import Graph
from .loss import softmax_cross_entropy_accuracy, softmax_cross_entropy_loss
from .module import (
    Conv2D,
    Dense,
    Dropout,
    EvalContext,
    Initializer,
    LSTMCell,
    MaxBlurPool2D,
    MaxPool2D,
    Module,
)
from .optimizer import Adam, StochasticGradientDescent, add_weight_decay_to_grad
from .shape import Shape, View

__all__ = [
    "Array", "DualArray", "Parameter", "Scope", "Environment", "Graph",
    "softmax_cross_entropy_accuracy", "softmax_cross_entropy_loss",
    "Conv2D", "Dense", "Dropout", "EvalContext", "Initializer", "LSTMCell", "MaxBlurPool2D", "MaxPool2D", "Module",
    "Adam", "StochasticGradientDescent", "add_weight_decay_to_grad", "Shape", "View",
]
