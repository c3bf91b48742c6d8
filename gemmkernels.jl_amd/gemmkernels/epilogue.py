"""Epilogues: the store of the D tile (reference src/epilogue.jl)."""
from __future__ import annotations

DEFAULT, BIAS, BIAS_ROW = range(3)


class Default:
    """src/epilogue.jl:14-34"""
    kind = DEFAULT
    bias = None

    def __repr__(self):
        return "Epilogue.Default()"


class Bias:
    """src/epilogue.jl:40-73: adds ``bias[j]`` (one fp32 value per COLUMN j of D) before the
    shared_to_global_d transform.  ``bias_pointer`` is a device pointer (int) or a CUDA tensor."""
    kind = BIAS

    def __init__(self, bias_pointer):
        self.bias = bias_pointer

    def __repr__(self):
        return "Epilogue.Bias(...)"


class BiasRow(Bias):
    """Adds ``bias[i]`` (one value per ROW i of D); no counterpart in the reference."""
    kind = BIAS_ROW

    def __repr__(self):
        return "Epilogue.BiasRow(...)"
