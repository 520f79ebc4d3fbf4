"""MI355X-native (gfx950) implementation of NestQuant's packed W4A4KV4 execution path.

Host code is Python on PyTorch-ROCm; every kernel lives in libnqhip.so behind the C ABI
declared in include/nqhip.h.  Sub-packages mirror the reference's module layout for the
path (core containers, runtime operators, the fused Linear module).
"""

__version__ = "0.1.0"
