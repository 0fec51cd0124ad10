"""cattle-hip: MI355X (gfx950) kernels for C-ATTL3's kernel-layer hot path.

The product is libcattle_hip.so (C ABI in include/cattle_hip.h, sources in csrc/). This package
is the Python binding used by the tests and the benchmark; the directory name is not a valid
identifier, so load it with importlib.import_module("c-attl3_amd").
"""
from .binding import *  # noqa: F401,F403
from .binding import build, lib, init, synchronize, trim, memory_info, EXPORTS, LIB_PATH, CattleHipError  # noqa: F401
