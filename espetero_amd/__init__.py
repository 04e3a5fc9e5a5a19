"""MI355X-native paged-KV attention: Python harness over the C ABI.

The product is the C-ABI library (csrc/, include/espetero_attn.h) and the C++
host engine (engine/). This package only loads them with ctypes and moves
torch device pointers across; it holds no arithmetic of its own.
"""
from . import abi  # noqa: F401
