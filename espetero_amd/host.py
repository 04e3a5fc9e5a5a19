"""ctypes binding of the host engine (include/espetero_engine.h): tile planner,
KV block pool, slots and the pass builder. Host memory only."""
import ctypes as C
import os

import numpy as np

from . import abi


class PlanOptions(C.Structure):
    _fields_ = [("rows_per_tile", C.c_int32), ("groups_target", C.c_int32), ("split", C.c_int32),
                ("min_chunk", C.c_int32), ("granule", C.c_int32), ("max_splits", C.c_int32),
                ("min_span", C.c_int32), ("balanced", C.c_int32), ("item_steps", C.c_int32), ("part_steps", C.c_int32),
                ("cut_batch", C.c_int32)]


class TreeSpec(C.Structure):
    _fields_ = [("parent", C.c_int32), ("save", C.c_int32), ("work", C.c_int32), ("root_len", C.c_int32),
                ("save_len", C.c_int32), ("n_leaves", C.c_int32), ("leaf_offsets", C.POINTER(C.c_int32)),
                ("leaf_tokens", C.POINTER(C.c_int32)), ("commit_chain", C.c_int32), ("noncausal", C.c_int32)]


_V, _I = C.c_void_p, C.c_int32
_ERR = (C.c_char_p, C.c_size_t)
_PO = C.POINTER(PlanOptions)
_TS = C.POINTER(TreeSpec)
_IP = C.POINTER(C.c_int32)
ENGINE_SYMBOLS = {
    "esp_plan_options_reference": (None, (_PO,)),
    "esp_plan_options_mi355x": (None, (_PO, _I, _I)),
    "esp_plan_tiles": (C.c_int, (_V, _I, _I, _I, _V, _PO, _V, _I, _IP, _V, _I, _IP, _IP) + _ERR),
    "esp_engine_create": (_V, (_I, _I, _I, _I)),
    "esp_engine_destroy": (None, (_V,)),
    "esp_engine_slot_alloc": (C.c_int, (_V,)),
    "esp_engine_slot_free": (C.c_int, (_V, _I)),
    "esp_engine_slot_reset": (C.c_int, (_V, _I)),
    "esp_engine_slot_fork": (C.c_int, (_V, _I, _I)),
    "esp_engine_slot_adopt": (C.c_int, (_V, _I, _I, _I)),
    "esp_engine_slot_len": (C.c_int, (_V, _I)),
    "esp_engine_slot_blocks": (C.c_int, (_V, _I, _V, _I)),
    "esp_engine_slot_next_pos": (C.c_int, (_V, _I)),
    "esp_engine_slot_chain": (C.c_int, (_V, _I)),
    "esp_engine_chain_commit": (C.c_int, (_V, _I, _I) + _ERR),
    "esp_engine_free_blocks": (C.c_int, (_V,)),
    "esp_engine_block_ref": (C.c_int, (_V, _I)),
    "esp_engine_pass_blocks": (C.c_int, (_V, _TS, _I)),
    "esp_engine_pass_begin": (C.c_int, (_V, _TS, _I) + _ERR),
    "esp_engine_pass_rows": (C.c_int, (_V,)),
    "esp_engine_pass_counts": (C.c_int, (_V, _IP, _IP, _IP)),
    "esp_engine_pass_trees": (C.c_int, (_V, _V)),
    "esp_engine_pass_desc": (C.c_int, (_V, _V)),
    "esp_engine_pass_pos": (C.c_int, (_V, _V)),
    "esp_engine_pass_table": (C.c_int, (_V, _V)),
    "esp_engine_pass_saves": (C.c_int, (_V, _V)),
    "esp_engine_pass_cow": (C.c_int, (_V, _V)),
    "esp_engine_pass_rings": (C.c_int, (_V, _I, _I, _V, _V, _I, _IP, _V, _I, _IP) + _ERR),
    "esp_slot_file_save": (C.c_int, (C.c_char_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_uint64, _V)),
    "esp_slot_file_info": (C.c_int, (C.c_char_p, C.c_int32, _V, _V, _V, _V, _V)),
    "esp_slot_file_load": (C.c_int, (C.c_char_p, C.c_int32, _V, C.c_uint64)),
    "esp_slot_file_save_rings": (C.c_int, (C.c_char_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_uint64, _V, C.c_int32, C.c_int32,
                                            C.c_uint64, _V)),
    "esp_slot_file_info_rings": (C.c_int, (C.c_char_p, C.c_int32, _V, _V, _V, _V, _V, _V, _V, _V)),
    "esp_slot_file_load_rings": (C.c_int, (C.c_char_p, C.c_int32, _V, C.c_uint64, _V, C.c_uint64)),
    "esp_kv_row_table": (C.c_int, (_V, C.c_int32, C.c_int32, _V, C.c_char_p, C.c_size_t)),
    "esp_engine_pass_commit": (C.c_int, (_V,)),
    "esp_engine_pass_abort": (C.c_int, (_V,)),
}

_lib = None


def engine_lib():
    global _lib
    if _lib is None:
        if not os.path.exists(abi.ENGINE_LIB_PATH):
            raise abi.EspError(f"{abi.ENGINE_LIB_PATH} is not built (run __graft_entry__.build())")
        lib = C.CDLL(abi.ENGINE_LIB_PATH)
        for name, (res, args) in ENGINE_SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = list(args)
        _lib = lib
    return _lib


def options_reference():
    o = PlanOptions()
    engine_lib().esp_plan_options_reference(C.byref(o))
    return o


def options_mi355x(rows, workgroups):
    o = PlanOptions()
    engine_lib().esp_plan_options_mi355x(C.byref(o), rows, workgroups)
    return o


def plan_tiles(trees, groups, window, pos, options):
    """trees: TREE_DT array. Returns (tiles TILE_DT, jobs COMBINE_DT, n_parts)."""
    lib = engine_lib()
    trees = np.ascontiguousarray(trees, dtype=abi.TREE_DT)
    pos_a = None if pos is None else np.ascontiguousarray(pos, dtype=np.int32)
    err = C.create_string_buffer(256)
    nt, nj, npart = C.c_int32(0), C.c_int32(0), C.c_int32(0)
    rc = lib.esp_plan_tiles(trees.ctypes.data, len(trees), groups, window, None if pos_a is None else pos_a.ctypes.data,
                            C.byref(options), None, 0, C.byref(nt), None, 0, C.byref(nj), C.byref(npart), err, 256)
    if rc not in (0, 4):
        abi.check(rc, err)
    tiles = np.zeros(nt.value, abi.TILE_DT)
    jobs = np.zeros(nj.value, abi.COMBINE_DT)
    rc = lib.esp_plan_tiles(trees.ctypes.data, len(trees), groups, window, None if pos_a is None else pos_a.ctypes.data,
                            C.byref(options), tiles.ctypes.data, len(tiles), C.byref(nt), jobs.ctypes.data, len(jobs),
                            C.byref(nj), C.byref(npart), err, 256)
    abi.check(rc, err)
    return tiles, jobs, npart.value


def slot_file_save(path, length, next_pos, n_layers, blocks_kv):
    """blocks_kv: host array [n_layers][n_blocks][block elements] of storage bits in the reference's block layout."""
    kv = np.ascontiguousarray(blocks_kv)
    n_layers_, n_blocks = kv.shape[0], kv.shape[1]
    assert n_layers_ == n_layers
    block_bytes = kv[0, 0].nbytes if n_blocks else 0
    rc = engine_lib().esp_slot_file_save(str(path).encode(), length, next_pos, n_blocks, n_layers, block_bytes,
                                         kv.ctypes.data if kv.size else None)
    if rc != 0:
        raise abi.EspError(f"slot_file_save({path}) failed")


def slot_file_save_rings(path, length, next_pos, n_layers, blocks_kv, rings):
    """slot_file_save with the ring section: rings = host array [r_layers][r_blocks][block elements], the slot's ring of
    every sliding layer in ring order, reference block layout."""
    kv, rg = np.ascontiguousarray(blocks_kv), np.ascontiguousarray(rings)
    assert kv.shape[0] == n_layers
    n_blocks = kv.shape[1]
    rc = engine_lib().esp_slot_file_save_rings(str(path).encode(), length, next_pos, n_blocks, n_layers,
                                               kv[0, 0].nbytes if n_blocks else 0, kv.ctypes.data if kv.size else None,
                                               rg.shape[0], rg.shape[1], rg[0, 0].nbytes if rg.size else 0,
                                               rg.ctypes.data if rg.size else None)
    if rc != 0:
        raise abi.EspError(f"slot_file_save_rings({path}) failed")


def slot_file_load_rings(path, bt):
    """slot_file_load for files with or without a ring section: the same dict plus r_layers, r_blocks, rblock_bytes and
    rings = uint8 [r_layers][r_blocks][rblock_bytes]; None for a refused file."""
    v = [C.c_int32(0) for _ in range(4)]
    r = [C.c_int32(0) for _ in range(2)]
    bb, rbb = C.c_uint64(0), C.c_uint64(0)
    lib = engine_lib()
    if lib.esp_slot_file_info_rings(str(path).encode(), bt, *[C.byref(x) for x in v], C.byref(bb), *[C.byref(x) for x in r],
                                    C.byref(rbb)) != 0:
        return None
    length, next_pos, n_blocks, n_layers = (x.value for x in v)
    kv = np.zeros((n_layers, n_blocks, bb.value), np.uint8)
    rings = np.zeros((r[0].value, r[1].value, rbb.value), np.uint8)
    if lib.esp_slot_file_load_rings(str(path).encode(), bt, kv.ctypes.data if kv.size else None, kv.nbytes,
                                    rings.ctypes.data if rings.size else None, rings.nbytes) != 0:
        return None
    return dict(len=length, next_pos=next_pos, n_blocks=n_blocks, n_layers=n_layers, block_bytes=bb.value, kv=kv,
                r_layers=r[0].value, r_blocks=r[1].value, rblock_bytes=rbb.value, rings=rings)


def slot_file_load(path, bt):
    """Returns dict(len, next_pos, n_blocks, n_layers, block_bytes, kv = uint8 [n_layers][n_blocks][block_bytes]), or None
    for a file the loader refuses (slot_load's -1, src/model/model.mm:700-714)."""
    v = [C.c_int32(0) for _ in range(4)]
    bb = C.c_uint64(0)
    if engine_lib().esp_slot_file_info(str(path).encode(), bt, *[C.byref(x) for x in v], C.byref(bb)) != 0:
        return None
    length, next_pos, n_blocks, n_layers = (x.value for x in v)
    kv = np.zeros((n_layers, n_blocks, bb.value), np.uint8)
    if engine_lib().esp_slot_file_load(str(path).encode(), bt, kv.ctypes.data if kv.size else None, kv.nbytes) != 0:
        return None
    return dict(len=length, next_pos=next_pos, n_blocks=n_blocks, n_layers=n_layers, block_bytes=bb.value, kv=kv)


def open_ended(tiles, trees):
    """Tiles of a decode chain: every tile whose cached range ends at its tree's cached length P gets
    k1 = INT32_MAX, which the kernels read as "up to P as the device holds it now", so the same records
    serve every step of a chain that esp_chain_advance moves on."""
    tiles = np.array(tiles, dtype=abi.TILE_DT, copy=True)
    P = np.asarray(trees["P"])[tiles["tree"]]
    tiles["k1"] = np.where(tiles["k1"] == P, np.int32(2**31 - 1), tiles["k1"])
    return tiles


def row_table(saves, rows):
    """KVSAVE_DT records -> int32 [rows][4] = (block, position, block2, position2), -1 none."""
    saves = np.ascontiguousarray(saves, dtype=abi.KVSAVE_DT)
    out = np.zeros((max(rows, 1), 4), np.int32)
    err = C.create_string_buffer(256)
    rc = engine_lib().esp_kv_row_table(saves.ctypes.data if len(saves) else None, len(saves), rows, out.ctypes.data, err, 256)
    if rc != 0:
        raise abi.EspError(err.value.decode(errors="replace"))
    return out[:rows]


def make_spec(parent=-1, save=-1, work=-1, root_len=0, save_len=0, leaves=(), commit_chain=0, noncausal=0):
    """leaves: list of token lists. Keeps the arrays alive on the returned struct."""
    s = TreeSpec(parent, save, work, root_len, save_len, len(leaves), None, None, commit_chain, noncausal)
    if leaves:
        offs = np.zeros(len(leaves) + 1, np.int32)
        offs[1:] = np.cumsum([len(x) for x in leaves])
        toks = np.ascontiguousarray(np.concatenate([np.asarray(x, np.int32) for x in leaves]), dtype=np.int32)
        s._keep = (offs, toks)
        s.leaf_offsets = offs.ctypes.data_as(_IP)
        s.leaf_tokens = toks.ctypes.data_as(_IP)
    return s


class Engine:
    """KV pool + slots + pass builder (C++ KvEngine)."""

    def __init__(self, n_blocks, bt, n_slots, max_ctx=1 << 30):
        self.lib = engine_lib()
        self.h = self.lib.esp_engine_create(n_blocks, bt, n_slots, max_ctx)
        if not self.h:
            raise abi.EspError("esp_engine_create failed")
        self.bt = bt

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.esp_engine_destroy(self.h)
            self.h = None

    def slot_alloc(self):
        return self.lib.esp_engine_slot_alloc(self.h)

    def slot_free(self, s):
        return self.lib.esp_engine_slot_free(self.h, s)

    def slot_reset(self, s):
        return self.lib.esp_engine_slot_reset(self.h, s)

    def slot_fork(self, a, b):
        return self.lib.esp_engine_slot_fork(self.h, a, b)

    def slot_adopt(self, length, next_pos, n_blocks):
        """A fresh slot of `length` positions in n_blocks new blocks (a loaded checkpoint): the slot, -1 or -2."""
        return self.lib.esp_engine_slot_adopt(self.h, length, next_pos, n_blocks)

    def slot_len(self, s):
        return self.lib.esp_engine_slot_len(self.h, s)

    def slot_next_pos(self, s):
        return self.lib.esp_engine_slot_next_pos(self.h, s)

    def slot_chain(self, s):
        return self.lib.esp_engine_slot_chain(self.h, s)

    def chain_commit(self, s, n):
        """The first n chain rows the slot's last pass kept become part of the slot. Raises EspError when refused."""
        err = C.create_string_buffer(256)
        abi.check(self.lib.esp_engine_chain_commit(self.h, s, n, err, 256), err)

    def slot_blocks(self, s):
        n = self.lib.esp_engine_slot_blocks(self.h, s, None, 0)
        out = np.zeros(max(n, 1), np.int32)
        self.lib.esp_engine_slot_blocks(self.h, s, out.ctypes.data, n)
        return out[:n].copy()

    def free_blocks(self):
        return self.lib.esp_engine_free_blocks(self.h)

    def block_ref(self, b):
        return self.lib.esp_engine_block_ref(self.h, b)

    def pass_blocks(self, specs):
        arr = (TreeSpec * len(specs))(*specs)
        return self.lib.esp_engine_pass_blocks(self.h, arr, len(specs))

    def pass_begin(self, specs):
        """Returns dict(trees, desc, pos, table, saves, cow, M). Raises EspError on a refused pass."""
        arr = (TreeSpec * len(specs))(*specs)
        err = C.create_string_buffer(256)
        rc = self.lib.esp_engine_pass_begin(self.h, arr, len(specs), err, 256)
        abi.check(rc, err)
        nt, ns, nc = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        n = self.lib.esp_engine_pass_counts(self.h, C.byref(nt), C.byref(ns), C.byref(nc))
        M = self.lib.esp_engine_pass_rows(self.h)
        trees = np.zeros(n, abi.TREE_DT)
        desc = np.zeros((max(M, 1), 4), np.int32)
        pos = np.zeros((max(M, 1), 4), np.int32)
        table = np.zeros(max(nt.value, 1), np.int32)
        saves = np.zeros(max(ns.value, 1), abi.KVSAVE_DT)
        cow = np.zeros((max(nc.value, 1), 2), np.int32)
        self.lib.esp_engine_pass_trees(self.h, trees.ctypes.data)
        self.lib.esp_engine_pass_desc(self.h, desc.ctypes.data)
        self.lib.esp_engine_pass_pos(self.h, pos.ctypes.data)
        self.lib.esp_engine_pass_table(self.h, table.ctypes.data)
        self.lib.esp_engine_pass_saves(self.h, saves.ctypes.data)
        self.lib.esp_engine_pass_cow(self.h, cow.ctypes.data)
        return dict(trees=trees, desc=desc[:M], pos=pos[:M], table=table[:nt.value], saves=saves[:ns.value],
                    cow=cow[:nc.value], M=M)

    def pass_rings(self, window, ring_blocks):
        """The pending pass on sliding layers: dict(trees, saves, copies)."""
        n = self.lib.esp_engine_pass_counts(self.h, None, None, None)
        trees = np.zeros(max(n, 1), abi.TREE_DT)
        ns, nc = C.c_int32(0), C.c_int32(0)
        err = C.create_string_buffer(256)
        rc = self.lib.esp_engine_pass_rings(self.h, window, ring_blocks, trees.ctypes.data, None, 0, C.byref(ns), None, 0,
                                            C.byref(nc), err, 256)
        if rc not in (0, 4):
            abi.check(rc, err)
        saves = np.zeros(max(ns.value, 1), abi.KVSAVE_DT)
        copies = np.zeros((max(nc.value, 1), 2), np.int32)
        rc = self.lib.esp_engine_pass_rings(self.h, window, ring_blocks, trees.ctypes.data, saves.ctypes.data, ns.value,
                                            C.byref(ns), copies.ctypes.data, nc.value, C.byref(nc), err, 256)
        abi.check(rc, err)
        return dict(trees=trees[:n], saves=saves[:ns.value], copies=copies[:nc.value])

    def pass_commit(self):
        return self.lib.esp_engine_pass_commit(self.h)

    def pass_abort(self):
        return self.lib.esp_engine_pass_abort(self.h)
