"""Pool maintenance through the C ABI: bit-exact against the checker's
reference-layout pool (index and page gathering carry no tolerance)."""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, synth
from oracle import binding as ob

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("HD,Hkv,bt,dtype", [(128, 4, 16, abi.ESP_F16), (256, 2, 16, abi.ESP_F16), (128, 8, 64, abi.ESP_BF16),
                                             (512, 2, 16, abi.ESP_F16), (512, 1, 64, abi.ESP_BF16)])
def test_relayout_gather_save_copy_are_bit_exact(HD, Hkv, bt, dtype):
    from gpu_utils import dev_u16, to_host_u16
    device.init(0)
    rng = np.random.default_rng(7)
    p = synth.make_params(Hkv * 2, Hkv, HD, dtype, bt)
    n_blocks, n_layers = 24, 3
    blk2 = 2 * bt * p.kv_ld
    region = n_blocks * blk2
    ref = rng.integers(0, 65536, n_layers * region).astype(np.uint16)
    ref_d = dev_u16(ref)
    nat = torch.zeros_like(ref_d)
    back = torch.zeros_like(ref_d)
    for l in range(n_layers):   # regions are converted one at a time
        device.kv_relayout(p, ref_d[l * region:], abi.ESP_LAYOUT_REFERENCE, nat[l * region:], abi.ESP_LAYOUT_NATIVE, n_blocks)
        device.kv_relayout(p, nat[l * region:], abi.ESP_LAYOUT_NATIVE, back[l * region:], abi.ESP_LAYOUT_REFERENCE, n_blocks)
    torch.cuda.synchronize()
    assert (to_host_u16(back) == ref).all()
    assert not (to_host_u16(nat) == ref).all()       # the native layout really is different

    # page walk: gather == the checker's gather, for a shuffled table
    table = rng.permutation(n_blocks).astype(np.int32)[:9]
    n_tok = 9 * bt - 5
    p.kv_base = region          # layer 1
    Kd = torch.zeros(n_tok * p.kv_ld, dtype=torch.int16, device="cuda")
    Vd = torch.zeros_like(Kd)
    device.kv_gather(p, nat, device.to_dev(table), n_tok, Kd, Vd)
    torch.cuda.synchronize()
    Kw, Vw = ob.kv_gather(p, ref, table, n_tok)
    assert (to_host_u16(Kd).reshape(n_tok, -1) == Kw).all() and (to_host_u16(Vd).reshape(n_tok, -1) == Vw).all()

    # append rows, some into two slots (a row may be saved twice: forest.h:1737-1749)
    rows = 11
    Kb = rng.integers(0, 65536, (rows, p.kv_ld)).astype(np.uint16)
    Vb = rng.integers(0, 65536, (rows, p.kv_ld)).astype(np.uint16)
    ent = np.array([(r, int(table[(40 + r) // bt]), (40 + r) % bt, 0) for r in range(rows)] +
                   [(3, int(table[8]), 1, 0)], abi.KVSAVE_DT)
    device.kv_save(p, dev_u16(Kb), dev_u16(Vb), nat, device.to_dev(ent), len(ent))
    ob.kv_save(p, Kb, Vb, ref, ent)
    # a prefill-like append: 40 consecutive rows from a 16-aligned token on (two whole sub-blocks through the
    # staged path, a ragged tail through element stores), source rows in reverse order
    rows2 = 40
    Kb2 = rng.integers(0, 65536, (rows2, p.kv_ld)).astype(np.uint16)
    Vb2 = rng.integers(0, 65536, (rows2, p.kv_ld)).astype(np.uint16)
    ent2 = np.array([(rows2 - 1 - r, int(table[(64 + r) // bt]), (64 + r) % bt, 0) for r in range(rows2)], abi.KVSAVE_DT)
    device.kv_save(p, dev_u16(Kb2), dev_u16(Vb2), nat, device.to_dev(ent2), len(ent2))
    ob.kv_save(p, Kb2, Vb2, ref, ent2)
    # copy on write in every layer region
    p.kv_base = 0
    pairs = np.array([(int(table[0]), int(table[8])), (int(table[2]), 23 if 23 not in table[:9] else int(table[7]))], np.int32)
    device.kv_copy_blocks(p, nat, device.to_dev(pairs), len(pairs), n_layers, region)
    ob.kv_copy_blocks(p, ref, pairs, n_layers, region)
    for l in range(n_layers):
        device.kv_relayout(p, nat[l * region:], abi.ESP_LAYOUT_NATIVE, back[l * region:], abi.ESP_LAYOUT_REFERENCE, n_blocks)
    torch.cuda.synchronize()
    assert (to_host_u16(back) == ref).all()


def test_time_next_brackets_the_attention_kernel_only():
    """esp_attn_time_next: the two events take the attention kernel's own begin and end; the pair is used once."""
    import torch
    from espetero_amd import device, host, synth
    from gpu_utils import dev_u16, native_pool
    device.init(0)
    c = synth.c1_single_decode()
    p = c.params
    tiles, jobs, n_parts = host.plan_tiles(c.trees, device.plan_hint(p)[1], 0, None,
                                           host.options_mi355x(p.rows_per_tile, device.plan_hint(p)[0]))
    dp = device.DevicePass(p, c.trees, tiles, jobs, n_parts, c.n_rows, c.blocks, None, None)
    Q, Kb, Vb, pool = dev_u16(c.Q), dev_u16(c.Kb), dev_u16(c.Vb), native_pool(c)
    O = torch.zeros_like(Q)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    b.record()
    torch.cuda.synchronize()
    for _ in range(3):
        dp.run(Q, Kb, Vb, pool, O)
    device.time_next(a, b)
    dp.run(Q, Kb, Vb, pool, O)
    dp.run(Q, Kb, Vb, pool, O)      # no pending pair any more: must not touch the events
    torch.cuda.synchronize()
    us = a.elapsed_time(b) * 1e3
    assert 1.0 < us < 200.0, us


def test_slot_checkpoint_round_trip_through_a_file(tmp_path):
    """save -> load -> attention (src/model/model.mm:629-752): the blocks of a slot leave the native pool in the
    reference's block layout, logical order, layer-major; loaded into other blocks of another pool they give
    the same attention output bit for bit, and the file's payload is the checker's reference-layout pool."""
    from espetero_amd import host
    from gpu_utils import dev_u16, to_host_u16
    device.init(0)
    n_layers = 2
    cases = [synth.make_case("slot", 20 + l, 8, 2, 128, abi.ESP_F16, 16, [(333, 1)], rows_per_tile=1) for l in range(n_layers)]
    c0 = cases[0]
    p = c0.params
    nb = (333 + 15) // 16
    blocks = np.asarray(c0.blocks[:nb], np.int32)
    blk = 2 * p.bt * p.kv_ld
    region = c0.n_blocks * blk
    # a two-layer pool: layer l's region holds case l's blocks (same block ids in both layers, as in the reference)
    ref = np.zeros(n_layers * region, np.uint16)
    for l, c in enumerate(cases):
        assert c.n_blocks == c0.n_blocks
        dst = ref[l * region:(l + 1) * region].reshape(c0.n_blocks, blk)
        dst[blocks] = c.pool_ref.reshape(c.n_blocks, blk)[c.blocks[:nb]]     # logical block i lives in block blocks[i] of every layer
    pool = torch.zeros(n_layers * region, dtype=torch.int16, device="cuda")
    for l in range(n_layers):
        device.kv_relayout(p, dev_u16(ref[l * region:(l + 1) * region]), abi.ESP_LAYOUT_REFERENCE,
                           pool[l * region:(l + 1) * region], abi.ESP_LAYOUT_NATIVE, c0.n_blocks)
    # export, layer-major
    out = torch.zeros(n_layers, nb, blk, dtype=torch.int16, device="cuda")
    bd = dev_u16(blocks.view(np.uint16)).view(torch.int32)
    for l in range(n_layers):
        p.kv_base = l * region
        device.kv_export_blocks(p, pool, bd, nb, out[l])
    torch.cuda.synchronize()
    payload = to_host_u16(out)
    for l in range(n_layers):                                   # == the checker's blocks in logical order
        want = ref[l * region:(l + 1) * region].reshape(c0.n_blocks, blk)[blocks]
        assert np.array_equal(payload[l], want)
    path = tmp_path / "slot.ckpt"
    host.slot_file_save(path, 333, 333, n_layers, payload)
    got = host.slot_file_load(path, p.bt)
    assert got is not None and got["len"] == 333 and got["n_blocks"] == nb and got["n_layers"] == n_layers
    # import into other blocks of a fresh pool
    new_blocks = np.random.default_rng(3).permutation(c0.n_blocks).astype(np.int32)[:nb]
    pool2 = torch.zeros_like(pool)
    nbd = dev_u16(new_blocks.view(np.uint16)).view(torch.int32)
    kv = got["kv"].view(np.uint16).reshape(n_layers, nb, blk)
    for l in range(n_layers):
        p.kv_base = l * region
        device.kv_import_blocks(p, dev_u16(kv[l]), nbd, nb, pool2)
    torch.cuda.synchronize()
    # attention per layer over the original and the reloaded slot
    resident, groups = device.plan_hint(p)
    for l, c in enumerate(cases):
        p.kv_base = l * region
        tiles, jobs, n_parts = host.plan_tiles(c.trees, groups, 0, None, host.options_mi355x(1, resident))
        Q, Kb, Vb = dev_u16(c.Q), dev_u16(c.Kb), dev_u16(c.Vb)
        outs = []
        for pl, bl in ((pool, blocks), (pool2, new_blocks)):
            dp = device.DevicePass(p, c.trees, tiles, jobs, n_parts, c.n_rows, bl, None, None)
            O = torch.zeros_like(Q)
            dp.run(Q, Kb, Vb, pl, O)
            torch.cuda.synchronize()
            outs.append(O)
        assert torch.equal(outs[0], outs[1]) and bool(outs[0].any())
    p.kv_base = 0


def test_slot_file_ring_section_reloads_a_sliding_layer_bit_identically(tmp_path):
    """A slot's ring of a sliding layer leaves through esp_kv_export_blocks (its ring blocks in ring order), travels
    in the slot file's ring section (model.mm:664-669), and comes back into another slot's ring: the sliding
    layer's attention over the reloaded ring is bit-identical."""
    from espetero_amd import host
    from gpu_utils import dev_u16, native_pool, to_host_u16
    device.init(0)
    bt, window = 16, 100
    c = synth.make_case("ringfile", 31, 8, 2, 256, abi.ESP_F16, bt, [(50, 1), (777, 1), (300, 1)], window=window, ring_layer=True,
                        rows_per_tile=1)
    p = c.params
    rb = p.ring
    blk = 2 * bt * p.kv_ld
    pool = native_pool(c)
    slot, new_slot = 1, 2
    assert int(c.trees[slot]["table"]) == slot * rb
    mine = np.arange(slot * rb, (slot + 1) * rb, dtype=np.int32)
    out = torch.zeros(1, rb, blk, dtype=torch.int16, device="cuda")
    device.kv_export_blocks(p, pool, device.to_dev(mine), rb, out[0])
    torch.cuda.synchronize()
    rings = to_host_u16(out)
    assert np.array_equal(rings[0], c.pool_ref.reshape(c.n_blocks, blk)[mine])      # == the checker's ring blocks
    P = int(c.trees[slot]["P"])
    path = tmp_path / "ring.ckpt"
    full = np.zeros((1, (P + bt - 1) // bt, 64), np.uint16)       # stands for the full-attention layers' blocks: the header's length must fit them
    host.slot_file_save_rings(path, P, P, 1, full, rings)
    got = host.slot_file_load_rings(path, bt)
    assert got is not None and (got["len"], got["r_layers"], got["r_blocks"], got["rblock_bytes"]) == (P, 1, rb, blk * 2)
    pool2 = torch.zeros_like(pool)
    theirs = np.arange(new_slot * rb, (new_slot + 1) * rb, dtype=np.int32)
    device.kv_import_blocks(p, dev_u16(got["rings"].view(np.uint16).reshape(1, rb, blk)[0]), device.to_dev(theirs), rb, pool2)
    torch.cuda.synchronize()
    # the sequence alone, from its own ring and from the reloaded one
    row = int(c.trees[slot]["base"])
    Q, Kb, Vb = (dev_u16(x[row:row + 1]) for x in (c.Q, c.Kb, c.Vb))
    pos = np.ascontiguousarray(c.pos.reshape(-1, 4)[row:row + 1])
    resident, groups = device.plan_hint(p)
    outs = []
    for pl, tab in ((pool, slot * rb), (pool2, new_slot * rb)):
        trees = np.array([(0, P, tab, 1)], abi.TREE_DT)
        tiles, jobs, n_parts = host.plan_tiles(trees, groups, window, pos, host.options_mi355x(1, resident))
        dp = device.DevicePass(p, trees, tiles, jobs, n_parts, 1, np.zeros(1, np.int32), None, pos)
        O = torch.zeros_like(Q)
        dp.run(Q, Kb, Vb, pl, O)
        torch.cuda.synchronize()
        outs.append(O)
    assert torch.equal(outs[0], outs[1]) and bool(outs[0].any())
