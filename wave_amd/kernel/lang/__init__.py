"""Element types and address spaces named by the scaled-GEMM templates
(``import wave_lang.kernel.lang as tkl`` in the reference)."""

from __future__ import annotations

import torch


class DataType:
    """Element type token (reference: wave_lang/kernel/_support/dtype.py)."""

    def __init__(self, name: str, torch_dtype):
        self.name = name
        self.torch_dtype = torch_dtype

    def __repr__(self):
        return f"DataType({self.name})"


f32 = DataType("f32", torch.float32)
bf16 = DataType("bf16", torch.bfloat16)
i8 = DataType("i8", torch.int8)
f4e2m1fn = DataType("f4E2M1FN", None)
f8e8m0fnu = DataType("f8E8M0FNU", None)


class AddressSpace:
    """Where a template keeps an operand.  The hand-written kernels fix this
    themselves (A and B through LDS, scales in registers); the tokens exist so
    template calls written for the reference keep working."""

    def __init__(self, name: str):
        self.name = name

    def __repr__(self):
        return f"AddressSpace({self.name})"


GLOBAL_ADDRESS_SPACE = AddressSpace("global")
SHARED_ADDRESS_SPACE = AddressSpace("shared")

TORCH_DTYPE_TO_WAVE = {torch.float32: f32, torch.bfloat16: bf16}
