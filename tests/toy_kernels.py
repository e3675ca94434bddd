"""Kernel modules that belong to test fixtures: registered with the engine's loader from outside the package,
as a part with a kernel of its own would register it."""
import os
from ctypes import c_float, c_int, c_void_p

from mini_inference_engine_amd.kernels.library import register_kernel_module

HERE = os.path.dirname(os.path.abspath(__file__))

register_kernel_module("toy_decay", {
    "toy_decay_scan": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p],
}, source=os.path.join(HERE, "toy_decay.hip"))
