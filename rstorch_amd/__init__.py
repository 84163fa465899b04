"""rstorch_amd: MI355X (gfx950) backend for the rstorch f64 training step.

The crate-root re-exports of the reference (src/lib.rs:10-14, 53-69) under the same names:
``Identity, Linear, ReLU, Sequential, CrossEntropyLoss, SGD`` plus the traits ``Module``,
``Loss``, ``Optimizer``, ``InitParameters`` and the ``sequential`` builder for the macro.
Everything computes on the GPU through ``librstorch_hip.so`` (``include/rstorch_hip.h``); there
is no CPU path in this package.
"""
from ._ffi import NanError, RstorchError, ShapeError, StateError
from .engine import Array2, Engine, as_array2, default_engine
from .init import FromArrays, InitParameters, KaimingNormal, Normal, XavierNormal
from .loss import CrossEntropyLoss, Loss
from .model import BasicModel, BatchStager, DeviceModel
from .module import (Identity, Linear, Module, Parameter, Parameters, ReLU, Sequential,
                     Softmax, sequential)
from .optim import SGD, Optimizer
from .utils import accuracy

__all__ = [
    "Array2", "Engine", "as_array2", "default_engine",
    "Module", "Parameter", "Parameters", "Identity", "Linear", "ReLU", "Softmax", "Sequential", "sequential",
    "Loss", "CrossEntropyLoss", "Optimizer", "SGD",
    "InitParameters", "KaimingNormal", "XavierNormal", "Normal", "FromArrays",
    "BasicModel", "DeviceModel", "BatchStager", "accuracy",
    "RstorchError", "ShapeError", "StateError", "NanError",
]
