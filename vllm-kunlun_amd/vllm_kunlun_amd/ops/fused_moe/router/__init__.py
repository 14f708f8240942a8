from .gate_linear import GateLinear  # noqa: F401
