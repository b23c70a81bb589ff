"""Schedule getters of the reference
(wave_lang/kernel/wave/schedules/gemm_mxfp4_double_buffer.py:42,284,519,726,
1102,1471,1781).  There they build a software-pipelining recipe for the
compiler; here the pipelining is fixed inside the hand-written kernels, so
each getter returns a token that ``wave_compile`` accepts and records."""

from __future__ import annotations

from dataclasses import dataclass, field


@dataclass(frozen=True)
class Schedule:
    name: str
    options: dict = field(default_factory=dict)


def get_mxfp4_dbuf_schedule(use_stagger: bool = True, k_partitions: int = 2):
    return Schedule("mxfp4_dbuf", {"use_stagger": use_stagger, "k_partitions": k_partitions})


def get_mxfp4_dbuf_pingpong_schedule(use_stagger: bool = True, shape=None, block_shape=None):
    return Schedule("mxfp4_dbuf_pingpong", {"use_stagger": use_stagger})


def get_mxfp4_dbuf_pingpong_schedule_Bshuffled(use_stagger: bool = True, shape=None, block_shape=None):
    return Schedule("mxfp4_dbuf_pingpong_Bshuffled", {"use_stagger": use_stagger})


def get_mxfp4_dbuf_pingpong_schedule_Bshuffled_lds(use_stagger: bool = True, shape=None, block_shape=None):
    return Schedule("mxfp4_dbuf_pingpong_Bshuffled_lds", {"use_stagger": use_stagger})


def get_mxfp4_dbuf_mixed_pingpong_schedule(use_stagger: bool = True):
    return Schedule("mxfp4_dbuf_mixed_pingpong", {"use_stagger": use_stagger})


def get_mxfp4_dbuf_mixed_pingpong_shuffle_schedule(use_stagger: bool = True):
    return Schedule("mxfp4_dbuf_mixed_pingpong_shuffle", {"use_stagger": use_stagger})


def get_mxfp4_asymmetric_schedule(eliminate_epilogue: bool = False, is_bscale_shuffled: bool = True):
    return Schedule("mxfp4_asymmetric", {"eliminate_epilogue": eliminate_epilogue,
                                        "is_bscale_shuffled": is_bscale_shuffled})
