"""ctypes view of the C ABI declared in include/espetero_attn.h.

The records mirror the reference's kernel-side structs field for field
(src/model/impl/forest.h:1308-1319, src/model/impl/gemma.h:29-35), so plans
built here can be compared with the reference's formulas directly.
"""
import ctypes as C
import os

import numpy as np

ESP_F16, ESP_BF16 = 0, 1
ESP_LAYOUT_REFERENCE, ESP_LAYOUT_NATIVE = 0, 1
ESP_ABI_VERSION = 3
ESP_PASS_FUSED, ESP_PASS_ROWS_IN_POOL = 1, 2
ESP_STATIC_SCRATCH_BYTES = 32 << 20

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ATTN_LIB_PATH = os.path.join(_PKG_DIR, "csrc", "libespetero_attn.so")
ENGINE_LIB_PATH = os.path.join(_PKG_DIR, "engine", "libespetero_engine.so")


class Tree(C.Structure):
    _fields_ = [("base", C.c_int32), ("P", C.c_int32), ("table", C.c_int32), ("M", C.c_int32)]


class Tile(C.Structure):
    _fields_ = [("tree", C.c_int32), ("r0", C.c_int32), ("k0", C.c_int32), ("k1", C.c_int32),
                ("part", C.c_int32), ("last", C.c_int32), ("b0", C.c_int32), ("pad", C.c_int32)]


class Combine(C.Structure):
    _fields_ = [("r0", C.c_int32), ("rows", C.c_int32), ("part0", C.c_int32), ("nparts", C.c_int32)]


class KVSave(C.Structure):
    _fields_ = [("src_row", C.c_int32), ("block", C.c_int32), ("pos", C.c_int32), ("pad", C.c_int32)]


class AttnParams(C.Structure):
    _fields_ = [("H", C.c_int32), ("Hkv", C.c_int32), ("head_dim", C.c_int32), ("dtype", C.c_int32),
                ("q_ld", C.c_int32), ("kv_ld", C.c_int32), ("bt", C.c_int32), ("window", C.c_int32),
                ("ring", C.c_int32), ("bidi", C.c_int32), ("rows_per_tile", C.c_int32), ("scale", C.c_float),
                ("kv_base", C.c_uint64), ("gate", C.c_void_p), ("gate_ld", C.c_int32), ("gate_hs", C.c_int32),
                ("gate_off", C.c_int32), ("gate_headwise", C.c_int32)]


class PrepParams(C.Structure):
    _fields_ = [("H", C.c_int32), ("Hkv", C.c_int32), ("head_dim", C.c_int32), ("dtype", C.c_int32),
                ("x_ld", C.c_int32), ("q_off", C.c_int32), ("q_hs", C.c_int32), ("k_off", C.c_int32),
                ("v_off", C.c_int32), ("q_ld", C.c_int32), ("kv_ld", C.c_int32), ("rope_dims", C.c_int32),
                ("v_norm", C.c_int32), ("bt", C.c_int32), ("eps", C.c_float), ("q_scale", C.c_float),
                ("kv_base", C.c_uint64)]


class GateParams(C.Structure):
    _fields_ = [("H", C.c_int32), ("head_dim", C.c_int32), ("D", C.c_int32), ("dtype", C.c_int32),
                ("q_ld", C.c_int32), ("x_ld", C.c_int32)]


TREE_DT = np.dtype([("base", "<i4"), ("P", "<i4"), ("table", "<i4"), ("M", "<i4")])
TILE_DT = np.dtype([("tree", "<i4"), ("r0", "<i4"), ("k0", "<i4"), ("k1", "<i4"),
                    ("part", "<i4"), ("last", "<i4"), ("b0", "<i4"), ("pad", "<i4")])
COMBINE_DT = np.dtype([("r0", "<i4"), ("rows", "<i4"), ("part0", "<i4"), ("nparts", "<i4")])
KVSAVE_DT = np.dtype([("src_row", "<i4"), ("block", "<i4"), ("pos", "<i4"), ("pad", "<i4")])

assert C.sizeof(Tree) == TREE_DT.itemsize == 16
assert C.sizeof(Tile) == TILE_DT.itemsize == 32
assert C.sizeof(Combine) == COMBINE_DT.itemsize == 16
assert C.sizeof(KVSave) == KVSAVE_DT.itemsize == 16
assert C.sizeof(AttnParams) == 80
assert C.sizeof(PrepParams) == 72
assert C.sizeof(GateParams) == 24

# name -> (restype, argtypes); every symbol the header declares.
_P = C.POINTER(AttnParams)
_V = C.c_void_p
_ERR = (C.c_char_p, C.c_size_t)
ATTN_SYMBOLS = {
    "esp_attn_init": (C.c_int, (C.c_int,) + _ERR),
    "esp_attn_abi_version": (C.c_int, ()),
    "esp_attn_plan_hint": (C.c_int, (_P, C.c_int, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)) + _ERR),
    "esp_attn_workspace_bytes": (C.c_size_t, (_P, C.c_int32, C.c_int32)),
    "esp_attn_forward": (C.c_int, (_P, _V, _V, _V, _V, _V, _V, _V, _V, _V, C.c_int32, _V, C.c_int32, _V, C.c_int32,
                                   C.c_int32, C.c_int32, _V, C.c_size_t, _V) + _ERR),
    "esp_attn_forward_static": (C.c_int, (_P, _V, _V, _V, _V, _V, _V, _V, _V, _V, C.c_int32, _V, C.c_int32, _V, C.c_int32,
                                          C.c_int32, C.c_int32, _V) + _ERR),
    "esp_attn_validate": (C.c_int, (_P, _V, C.c_int32, _V, C.c_int32, _V, C.c_int32, C.c_int32, C.c_int32, _V, C.c_int32,
                                    C.c_int32) + _ERR),
    "esp_attn_validate_for": (C.c_int, (_P, C.c_int32, _V, C.c_int32, _V, C.c_int32, _V, C.c_int32, C.c_int32, C.c_int32, _V, C.c_int32,
                                        C.c_int32) + _ERR),
    "esp_attn_time_next": (C.c_int, (_V, _V)),
    "esp_attn_combine": (C.c_int, (_P, _V, _V, C.c_int32, C.c_int32, C.c_int32, _V, C.c_size_t, _V) + _ERR),
    "esp_kv_save": (C.c_int, (_P, _V, _V, _V, _V, C.c_int32, _V) + _ERR),
    "esp_kv_copy_blocks": (C.c_int, (_P, _V, _V, C.c_int32, C.c_int32, C.c_uint64, _V) + _ERR),
    "esp_kv_gather": (C.c_int, (_P, _V, _V, C.c_int32, _V, _V, _V) + _ERR),
    "esp_kv_relayout": (C.c_int, (_P, _V, C.c_int32, _V, C.c_int32, C.c_int32, _V) + _ERR),
    "esp_kv_export_blocks": (C.c_int, (_P, _V, _V, C.c_int32, _V, _V) + _ERR),
    "esp_kv_import_blocks": (C.c_int, (_P, _V, _V, C.c_int32, _V, _V) + _ERR),
    "esp_chain_advance": (C.c_int, (_V, C.c_int32, _V, _V, _V, C.c_int32, C.c_int32, _V) + _ERR),
    "esp_head_gate": (C.c_int, (C.POINTER(GateParams), _V, _V, _V, _V, C.c_int32, _V) + _ERR),
    "esp_attn_decode_fused": (C.c_int, (C.POINTER(PrepParams), _P, _V, _V, _V, _V, _V, _V, _V, _V, _V, _V, _V, _V, C.c_int32, _V, C.c_int32,
                                        _V, C.c_int32, C.c_int32, C.c_int32, _V, C.c_size_t, _V) + _ERR),
    "esp_attn_prep": (C.c_int, (C.POINTER(PrepParams), _V, _V, _V, _V, _V, _V, _V, _V, _V, _V, _V, C.c_int32, _V) + _ERR),
}


class EspError(RuntimeError):
    pass


_attn_lib = None


def attn_lib():
    """The HIP library. There is no fallback: a missing build is an error."""
    global _attn_lib
    if _attn_lib is None:
        if not os.path.exists(ATTN_LIB_PATH):
            raise EspError(f"{ATTN_LIB_PATH} is not built (run __graft_entry__.build())")
        lib = C.CDLL(ATTN_LIB_PATH)
        for name, (res, args) in ATTN_SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = list(args)
        if lib.esp_attn_abi_version() != ESP_ABI_VERSION:
            raise EspError("libespetero_attn.so: ABI version mismatch")
        _attn_lib = lib
    return _attn_lib


def check(rc, errbuf):
    if rc != 0:
        raise EspError(f"esp error {rc}: {errbuf.value.decode(errors='replace')}")
