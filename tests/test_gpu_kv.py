"""Pool maintenance through the C ABI: bit-exact against the checker's
reference-layout pool (index and page gathering carry no tolerance)."""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, synth
from oracle import binding as ob

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("HD,Hkv,bt,dtype", [(128, 4, 16, abi.ESP_F16), (256, 2, 16, abi.ESP_F16), (128, 8, 64, abi.ESP_BF16)])
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
