"""MI355X (gfx950) back end for rust-model-inference's quantized matrix products.

``synth``  seeded synthetic tensors of the benchmark shapes (numpy only)
``gguf``   minimal GGUF v3 writer / mmap reader (synthetic Qwen3 file)
``hip``    ctypes binding of librmi_hip.so, the C ABI of include/rmi_hip.h
``kernel`` mirror of the reference's Kernel / Layer interface over that ABI
``decode`` mirror of Qwen3Session over the device-resident decode entry points
``loader`` mirror of GGUFLoader over the library's parser; file -> HBM uploads

``hip``, ``kernel``, ``decode`` and ``loader`` load the compiled library on first use and raise if it
is missing; nothing here computes on the CPU.
"""
import importlib

from . import gguf, synth  # noqa: F401

_LAZY = ("hip", "kernel", "decode", "loader")


def __getattr__(name):
    if name in _LAZY:
        return importlib.import_module(f"{__name__}.{name}")
    if name == "init":
        return importlib.import_module(f"{__name__}.hip").init
    raise AttributeError(name)
