"""MI355X-native tensor backend for catgrad's Interpreter.

The product is csrc/ (HIP kernels for gfx950 + the C++ host runtime behind the C ABI of
include/catgrad_hip.h).  The Python modules are the host-side mirror of the reference's
caller: `abi` binds the C ABI, `lang`/`nn` restate the graph DSL, `interpreter` marshals
values for the native evaluator, `llm` holds the model definitions.
"""
from . import abi, lang, nn, interpreter  # noqa: F401
from .abi import (Backend, Tensor, BackendPanic, ShapeError, InterpreterError, load_library,
                  F32, U32, FLAG_BF16, FLAG_EAGER, FLAG_NO_PATTERNS)  # noqa: F401
from .interpreter import (Interpreter, Environment, Parameters, WeightFile, WeightsError, stdlib,  # noqa: F401
                          tensor)
