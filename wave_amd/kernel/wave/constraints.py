"""Scaled MFMA variants (wave_lang/kernel/wave/constraints.py:79-85)."""

from enum import Enum


class ScaledMMAType(Enum):
    # Intrinsics introduced in CDNA4
    F32_16x16x128_F8F6F4 = 0x1340
    F32_32x32x64_F8F6F4 = 0x1341
