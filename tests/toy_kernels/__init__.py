"""Kernel files that toy parts of the tests bring along, registered with the package's build."""

import ctypes
import os

from burn_transformers_amd.kernels import library as K

HERE = os.path.dirname(os.path.abspath(__file__))


class RotaryTurnCall(ctypes.Structure):
    """Mirror of the structure in rotary_turn.hip."""
    _fields_ = [("dtype", ctypes.c_int), ("tokens", ctypes.c_int), ("parts", ctypes.c_int), ("heads", ctypes.c_int),
                ("head_dim", ctypes.c_int), ("ld", ctypes.c_int64), ("rows", ctypes.c_void_p),
                ("positions", ctypes.c_void_p), ("freq", ctypes.c_void_p)]
    # the field that holds a step's number of tokens: with it said, a launch list that holds such a
    # call serves every step of its class, not only the one it was recorded for
    _step_fields_ = {"tokens": "tokens"}


def register():
    """Makes the toy modules known to the package's build; returns their names."""
    K.register_module("toy_rotary_turn", os.path.join(HERE, "rotary_turn.hip"))
    return ["toy_rotary_turn"]
