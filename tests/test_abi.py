"""The C-ABI libraries load and export every symbol the headers declare.
No compute calls: these run without a GPU."""
import ctypes as C
import os
import re

from espetero_amd import abi, host

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(esp_[a-z0-9_]+)\s*\(", text)))


def test_attn_library_exports_every_declared_symbol():
    names = _declared("espetero_attn.h")
    assert set(names) == set(abi.ATTN_SYMBOLS), "the ctypes table must name exactly what the header declares"
    lib = C.CDLL(abi.ATTN_LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    lib.esp_attn_abi_version.restype = C.c_int
    assert lib.esp_attn_abi_version() == abi.ESP_ABI_VERSION


def test_engine_library_exports_every_declared_symbol():
    names = _declared("espetero_engine.h")
    assert set(names) == set(host.ENGINE_SYMBOLS)
    lib = C.CDLL(abi.ENGINE_LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n


def test_ceilings_library_exports_every_declared_symbol_and_refuses_bad_arguments():
    names = _declared("espetero_ceilings.h")
    assert names == ["esp_ceiling_hbm_read", "esp_ceiling_mfma_issue", "esp_ceiling_prefill_step", "esp_ceiling_prefill_step256"]
    lib = C.CDLL(os.path.join(ROOT, "espetero_amd", "csrc", "libespetero_ceilings.so"))
    for n in names:
        assert hasattr(lib, n), n
    V, I = C.c_void_p, C.c_int32
    lib.esp_ceiling_hbm_read.argtypes = [V, V, I, I, I, I, V, V, V, V]
    lib.esp_ceiling_mfma_issue.argtypes = [I, I, I, I, I, V, V, V, V]
    lib.esp_ceiling_prefill_step.argtypes = [I, I, I, I, I, V, V, V, V, V, V]
    assert lib.esp_ceiling_hbm_read(None, None, 4, 8192, 1, 8, None, None, None, None) == 1        # no buffer: refused on the host
    assert lib.esp_ceiling_mfma_issue(0, 0, 1, 8, 10, None, None, None, None) == 1
    assert lib.esp_ceiling_prefill_step(4, 1, 1, 8, 10, None, None, None, None, None, None) == 1
    lib.esp_ceiling_prefill_step256.argtypes = [I, I, I, I, V, V, V, V, V, V]
    assert lib.esp_ceiling_prefill_step256(0, 1, 8, 10, None, None, None, None, None, None) == 1


def test_record_layouts_match_the_reference_structs():
    """AttnTree 16 B, tile 32 B, combine 16 B, KVSave 16 B (kernels/40_attention.metal:134-150,
    804-809, 868-873): field order is part of the contract."""
    assert [f[0] for f in abi.Tree._fields_] == ["base", "P", "table", "M"]
    assert [f[0] for f in abi.Tile._fields_] == ["tree", "r0", "k0", "k1", "part", "last", "b0", "pad"]
    assert [f[0] for f in abi.Combine._fields_] == ["r0", "rows", "part0", "nparts"]
    assert [f[0] for f in abi.KVSave._fields_] == ["src_row", "block", "pos", "pad"]


def test_workspace_bytes_is_host_arithmetic():
    from espetero_amd import synth
    lib = abi.attn_lib()
    p = synth.make_params(32, 4, 128, abi.ESP_F16, 16, rows_per_tile=1)
    assert lib.esp_attn_workspace_bytes(C.byref(p), 16, 0) >= 1
    n = lib.esp_attn_workspace_bytes(C.byref(p), 16, 100)
    assert n >= 100 * 4 * 8 * (128 + 2) * 4          # parts x Hkv x packed rows x (O, m, l) floats
    p2 = synth.make_params(40, 8, 128, abi.ESP_BF16, 16, rows_per_tile=128)
    n2 = lib.esp_attn_workspace_bytes(C.byref(p2), 2048, 0)
    assert n2 >= 2048 * 8 * 128 * 2                   # the transposed staging copy of the batch V rows


def test_argument_errors_come_back_as_codes_not_crashes():
    """Checked on the host before any launch."""
    from espetero_amd import synth
    lib = abi.attn_lib()
    err = C.create_string_buffer(256)
    p = synth.make_params(32, 5, 128, abi.ESP_F16, 16)
    rc = lib.esp_attn_forward(C.byref(p), None, None, None, None, None, None, None, None, None, 1, None, 1, None, 0, 0, 1,
                              None, 0, None, err, 256)
    assert rc == 1 and b"multiple of Hkv" in err.value
    p = synth.make_params(32, 4, 96, abi.ESP_F16, 16)
    rc = lib.esp_kv_save(C.byref(p), None, None, None, None, 1, None, err, 256)
    assert rc == 2 and b"head_dim" in err.value
    p = synth.make_params(32, 4, 128, abi.ESP_F16, 24)
    rc = lib.esp_kv_gather(C.byref(p), None, None, 1, None, None, None, err, 256)
    assert rc == 1 and b"multiple of 16" in err.value
    p = synth.make_params(32, 4, 128, abi.ESP_F16, 16)
    rc = lib.esp_attn_forward(C.byref(p), None, None, None, None, None, None, None, None, None, 1, None, 1, None, 0, 0, 1,
                              None, 0, None, err, 256)
    assert rc == 1 and b"must not be NULL" in err.value


def test_prep_gate_and_chain_argument_errors():
    """The entry points beside the attention refuse bad arguments on the host too."""
    from espetero_amd import synth
    lib = abi.attn_lib()
    err = C.create_string_buffer(256)
    g, _ = synth.make_gate(16, 256, 2560, abi.ESP_F16, 1)
    assert lib.esp_head_gate(C.byref(g), None, None, None, None, 4, None, err, 256) == 1 and b"neither O nor dots" in err.value
    g.H = 65
    assert lib.esp_head_gate(C.byref(g), None, None, None, None, 4, None, err, 256) == 2 and b"1 .. 64" in err.value
    g.H, g.D = 16, 2564
    assert lib.esp_head_gate(C.byref(g), None, None, None, None, 4, None, err, 256) == 1 and b"multiple of 8" in err.value
    g.D, g.head_dim = 2560, 2048
    assert lib.esp_head_gate(C.byref(g), None, None, None, None, 4, None, err, 256) == 1 and b"at most 1024" in err.value
    g.head_dim = 256
    dots = (C.c_float * 64)()
    assert lib.esp_head_gate(C.byref(g), None, None, None, dots, 0, None, err, 256) == 0           # nothing to do
    assert lib.esp_head_gate(C.byref(g), None, None, None, dots, 4, None, err, 256) == 1 and b"X and Wg" in err.value
    p, _ = synth.make_prep("gemma", 8, 2, 128, abi.ESP_F16, 1)
    p.rope_dims = 48
    assert lib.esp_attn_prep(C.byref(p), None, None, None, None, None, None, None, None, None, None, None, 1, None, err, 256) == 1
    assert b"power of two" in err.value
    p.rope_dims, p.x_ld = 128, 100
    assert lib.esp_attn_prep(C.byref(p), None, None, None, None, None, None, None, None, None, None, None, 1, None, err, 256) == 1
    assert lib.esp_chain_advance(None, 3, None, None, None, 16, 0, None, err, 256) == 1 and b"trees and pos" in err.value
    assert lib.esp_chain_advance(None, 0, None, None, None, 16, 0, None, err, 256) == 0
    a = synth.make_params(32, 4, 128, abi.ESP_F16, 16)
    a.gate_headwise = 2
    assert lib.esp_attn_forward(C.byref(a), None, None, None, None, None, None, None, None, None, 1, None, 1, None, 0, 0, 1,
                                None, 0, None, err, 256) == 1 and b"gate_headwise" in err.value


def test_fused_decode_refuses_what_its_kernel_does_not_serve():
    """esp_attn_decode_fused: prep and attention parameters must agree, head dim 512 and tiles of more than 4 rows are
    refused with a message, all before any device call."""
    from espetero_amd import synth
    lib = abi.attn_lib()
    err = C.create_string_buffer(256)

    def call(pp, ap):
        return lib.esp_attn_decode_fused(C.byref(pp), C.byref(ap), None, None, None, None, None, None, None, None, None, None, None,
                                         None, 1, None, 1, None, 0, 0, 1, None, 0, None, err, 256)

    pp, _ = synth.make_prep("omni", 8, 2, 128, abi.ESP_F16, 1)
    ap = synth.make_params(8, 2, 128, abi.ESP_F16, 16, rows_per_tile=8)
    assert call(pp, ap) == 2 and b"1 to 4 rows" in err.value
    ap.rows_per_tile = 4
    assert call(pp, ap) == 1 and b"X, qn_w, kn_w" in err.value
    ap.Hkv, ap.kv_ld = 4, 512
    assert call(pp, ap) == 1 and b"different heads" in err.value
    pp, _ = synth.make_prep("gemma", 8, 1, 512, abi.ESP_F16, 1)
    ap = synth.make_params(8, 1, 512, abi.ESP_F16, 16, rows_per_tile=1)
    assert call(pp, ap) == 2 and b"128 and 256" in err.value
    pp, _ = synth.make_prep("gemma", 32, 2, 256, abi.ESP_F16, 1)
    ap = synth.make_params(32, 2, 256, abi.ESP_F16, 16, rows_per_tile=4)      # 4 rows x 16 heads per KV head: beyond the packed columns
    assert call(pp, ap) == 2


def _planned_pass():
    """A small decode + verify pass planned on the host: records as numpy arrays."""
    import numpy as np
    from espetero_amd import synth
    p = synth.make_params(32, 4, 128, abi.ESP_F16, 16, rows_per_tile=4)
    trees = np.array([(0, 1000, 0, 4), (4, 70, 63, 1), (5, 0, 68, 2)], abi.TREE_DT)
    tiles, jobs, n_parts = host.plan_tiles(trees, 4, 0, None, host.options_mi355x(4, 64))
    blocks = np.arange(63 + 5 + 1, dtype=np.int32)[::-1].copy()
    assert n_parts > 2 and len(jobs) >= 1
    return p, trees, tiles, jobs, n_parts, 7, blocks, 80


def test_validate_accepts_a_planned_pass_and_names_the_first_bad_record():
    """esp_attn_validate is host arithmetic over host copies of the records: every index a kernel would
    dereference, checked before the upload."""
    import numpy as np
    import pytest
    from espetero_amd import device
    p, trees, tiles, jobs, n_parts, n_rows, blocks, pool_blocks = _planned_pass()
    device.validate(p, tiles, trees, jobs, n_parts, n_rows, blocks, pool_blocks)
    device.validate(p, tiles, trees, jobs[:0], n_parts, n_rows, blocks, pool_blocks)   # merge as its own call: no jobs here

    def bad(match, tiles=tiles, trees=trees, jobs=jobs, n_parts=n_parts, n_rows=n_rows, blocks=blocks, pool_blocks=pool_blocks):
        with pytest.raises(abi.EspError, match=match):
            device.validate(p, tiles, trees, jobs, n_parts, n_rows, blocks, pool_blocks)

    i0 = int(np.flatnonzero(tiles["tree"] == 0)[0])   # a record of the first tree (4 rows, 1000 cached keys), wherever the planner lists it
    t = tiles.copy(); t[1]["tree"] = 3
    bad("tile 1: tree 3 of 3", tiles=t)
    t = tiles.copy(); t[i0]["part"] = n_parts
    bad(f"tile {i0}: partial record", tiles=t)
    t = tiles.copy(); t[i0]["r0"] = 4
    bad(f"tile {i0}: first row 4 outside", tiles=t)
    t = tiles.copy(); t[i0]["pad"] = 7
    bad(f"tile {i0}: pad 7", tiles=t)
    t = tiles.copy(); t[i0]["k1"] = 1001
    bad(f"tile {i0}: cached range", tiles=t)
    t = tiles.copy(); t[i0]["b0"] = 9
    bad("first batch key 9", tiles=t)
    split = [i for i in range(len(tiles)) if tiles[i]["part"] >= 0]
    t = tiles.copy(); t[split[1]]["part"] = t[split[0]]["part"]
    bad("written by another tile too", tiles=t)
    t = np.delete(tiles, split[0])
    bad("which no tile writes", tiles=t)
    tr = trees.copy(); tr[2]["M"] = 3
    bad("tree 2: rows", trees=tr)
    tr = trees.copy(); tr[0]["table"] = 10
    bad("tree 0: block list", trees=tr)
    b = blocks.copy(); b[5] = 80
    bad("tree 0: block 80", blocks=b)
    bad("tree 0: block 68", pool_blocks=68)
    j = jobs.copy(); j[0]["nparts"] += 1
    bad("job 0: parts|merged by jobs", jobs=j)
    j = jobs.copy(); j[0]["rows"] = 5
    bad("job 0: rows", jobs=j)
    j = np.concatenate([jobs, jobs[:1]])
    bad("merged by jobs 0 and", jobs=j)
    # ring layers: the tree's table is the first block of its slot's ring
    p.ring, p.window = 4, 64
    tr = np.array([(0, 1000, 8, 1)], abi.TREE_DT)
    tl, jb, npart = host.plan_tiles(tr, 4, 64, np.full((1, 4), 1000, np.int32), host.options_mi355x(1, 8))
    device.validate(p, tl, tr, jb, npart, 1, None, 12)
    with pytest.raises(abi.EspError, match="ring blocks"):
        device.validate(p, tl, tr, jb, npart, 1, None, 11)


def test_validate_fused_wants_one_tile_group_per_tree():
    """esp_attn_validate_fused: esp_attn_validate plus what esp_attn_decode_fused relies on and cannot see on the device:
    trees of at most rows_per_tile rows, each tile starting at its tree's first row."""
    import numpy as np
    import pytest
    from espetero_amd import device
    p, trees, tiles, jobs, n_parts, n_rows, blocks, pool_blocks = _planned_pass()
    device.validate(p, tiles, trees, jobs, n_parts, n_rows, blocks, pool_blocks, fused=True)   # trees of 4, 1 and 2 rows at 4 rows per tile
    p.rows_per_tile = 2                         # the first tree now needs two tile groups
    tl, jb, npart = host.plan_tiles(trees, 4, 0, None, host.options_mi355x(2, 64))
    device.validate(p, tl, trees, jb, npart, n_rows, blocks, pool_blocks)
    with pytest.raises(abi.EspError, match="tree 0: 4 rows"):
        device.validate(p, tl, trees, jb, npart, n_rows, blocks, pool_blocks, fused=True)
    p.rows_per_tile = 8
    tl, jb, npart = host.plan_tiles(trees, 4, 0, None, host.options_mi355x(8, 64))
    with pytest.raises(abi.EspError, match="fused decode takes trees of 1 to 4 rows"):
        device.validate(p, tl, trees, jb, npart, n_rows, blocks, pool_blocks, fused=True)


def test_validate_names_what_a_pass_without_kb_vb_has_to_promise():
    """ESP_PASS_ROWS_IN_POOL: block lists that reach P + M, P - base a multiple of 16 on the tiled kernel, no ring overrun."""
    import numpy as np
    import pytest
    from espetero_amd import device, synth
    opts = host.options_mi355x(128, 512)

    def case(seqs, **kw):   # block lists sized for P + M keys, of which P are cached
        c = synth.make_case("rows_in_pool", 64, 4, 2, 128, abi.ESP_F16, 16, [(P + M, M) for P, M in seqs], **kw)
        for t, (P, M) in zip(c.trees, seqs):
            t["P"] = P
        return c
    c = case([(48, 128), (208, 8)], rows_per_tile=128)   # P - base = 48 and 208 - 128 = 80; the second tree's rows open a block of their own
    tiles, jobs, n_parts = host.plan_tiles(c.trees, 4, 0, None, opts)
    device.validate(c.params, tiles, c.trees, jobs, n_parts, c.n_rows, c.blocks, c.n_blocks, rows_in_pool=True)
    with pytest.raises(abi.EspError, match="with its own rows appended"):
        device.validate(c.params, tiles, c.trees, jobs, n_parts, c.n_rows, c.blocks[:-1], c.n_blocks, rows_in_pool=True)
    c = case([(40, 130)], rows_per_tile=128)            # P - base = 40
    tiles, jobs, n_parts = host.plan_tiles(c.trees, 4, 0, None, opts)
    device.validate(c.params, tiles, c.trees, jobs, n_parts, c.n_rows, c.blocks, c.n_blocks)
    with pytest.raises(abi.EspError, match="no multiple of 16"):
        device.validate(c.params, tiles, c.trees, jobs, n_parts, c.n_rows, c.blocks, c.n_blocks, rows_in_pool=True)
    c.params.rows_per_tile = 4                          # the streaming kernel reads row by row: any P
    tiles, jobs, n_parts = host.plan_tiles(c.trees, 2, 0, None, host.options_mi355x(4, 512))
    device.validate(c.params, tiles, c.trees, jobs, n_parts, c.n_rows, c.blocks, c.n_blocks, rows_in_pool=True)
    c = synth.make_case("ring", 66, 4, 2, 128, abi.ESP_F16, 16, [(900, 40)], window=256, ring_layer=True, rows_per_tile=8)
    tiles, jobs, n_parts = host.plan_tiles(c.trees, 2, 256, c.pos, host.options_mi355x(8, 512))
    with pytest.raises(abi.EspError, match="overwrite keys"):
        device.validate(c.params, tiles, c.trees, jobs, n_parts, c.n_rows, None, c.n_blocks, rows_in_pool=True)
    c.trees[0]["M"] = 1
    tiles, jobs, n_parts = host.plan_tiles(c.trees, 2, 256, c.pos, host.options_mi355x(8, 512))
    device.validate(c.params, tiles, c.trees, jobs, n_parts, c.n_rows, None, c.n_blocks, rows_in_pool=True)


def test_validate_accepts_the_tiled_planner_s_partly_split_chunk():
    """A prefill chunk planned for the tiled kernel (128-row tiles, only the shortest tiles cut into parts of unequal
    count) passes the validator; dropping one of a tile's parts does not."""
    import numpy as np
    import pytest
    from espetero_amd import device, synth
    p = synth.make_params(40, 8, 128, abi.ESP_BF16, 16, rows_per_tile=128)
    trees = np.array([(0, 6144, 0, 2048)], abi.TREE_DT)
    tiles, jobs, n_parts = host.plan_tiles(trees, 40, 0, None, host.options_mi355x(128, 512))
    assert n_parts > 4 and len(jobs) == 4
    blocks = np.arange((6144 + 2048) // 16, dtype=np.int32)
    device.validate(p, tiles, trees, jobs, n_parts, 2048, blocks, len(blocks))
    with pytest.raises(abi.EspError, match="which no tile writes"):
        device.validate(p, np.delete(tiles, 1), trees, jobs, n_parts, 2048, blocks, len(blocks))


def test_forward_static_refuses_what_does_not_fit_its_scratch_array():
    """The entry point without a workspace names its limit; checked on the host before any launch or device call."""
    from espetero_amd import synth
    lib = abi.attn_lib()
    err = C.create_string_buffer(256)
    p = synth.make_params(32, 5, 128, abi.ESP_F16, 16)
    rc = lib.esp_attn_forward_static(C.byref(p), None, None, None, None, None, None, None, None, None, 1, None, 1, None, 0, 0, 1,
                                     None, err, 256)
    assert rc == 1 and b"multiple of Hkv" in err.value
    p = synth.make_params(32, 4, 128, abi.ESP_F16, 16, rows_per_tile=4)
    assert lib.esp_attn_workspace_bytes(C.byref(p), 32, 4096) > abi.ESP_STATIC_SCRATCH_BYTES
