"""Runs synthetic cases through the C ABI on the GPU (used by the -m gpu tests)."""
import numpy as np
import torch

from espetero_amd import abi, device, host


def dev_u16(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16).copy()).to("cuda")


def to_host_u16(t):
    return t.cpu().numpy().view(np.uint16)


def native_pool(case, nan_fill=False):
    """Device pool in the native layout, made from the case's reference-layout pool by esp_kv_relayout."""
    ref = dev_u16(case.pool_ref)
    nat = torch.empty_like(ref)
    device.kv_relayout(case.params, ref, abi.ESP_LAYOUT_REFERENCE, nat, abi.ESP_LAYOUT_NATIVE, case.n_blocks)
    torch.cuda.synchronize()
    return nat


def default_options(case, workgroups=None):
    return host.options_mi355x(case.params.rows_per_tile, workgroups or device.plan_hint(case.params)[0])


def plan(case, options):
    p = case.params
    p.rows_per_tile = options.rows_per_tile
    return host.plan_tiles(case.trees, device.plan_hint(p)[1], p.window, case.pos if p.window > 0 else None, options)


def append_rows(case, pool):
    """esp_kv_save of every tree's rows to positions P + j of the tree's own block list (or ring): what a pass whose
    attention reads its rows from the pool has had done before it."""
    p, bt = case.params, case.params.bt
    e = np.zeros(case.n_rows, abi.KVSAVE_DT)
    for t in case.trees:
        base, P, tab, M = int(t["base"]), int(t["P"]), int(t["table"]), int(t["M"])
        q = P + np.arange(M)
        e["src_row"][base:base + M] = base + np.arange(M)
        e["block"][base:base + M] = tab + (q // bt) % p.ring if p.ring else case.blocks[tab + q // bt]
        e["pos"][base:base + M] = q % bt
    device.kv_save(p, dev_u16(case.Kb), dev_u16(case.Vb), pool, device.to_dev(e), len(e))


def run_case(case, options=None, pool=None, with_desc=True, static=False, two_step=False, rows_in_pool=False):
    """Returns O as storage bits [n_rows][H * HD]. static: through esp_attn_forward_static (the library's own
    scratch array). two_step: attention with the merge left out, then esp_attn_combine as its own call.
    rows_in_pool: the pass's rows are appended to the pool first and the attention runs without Kb / Vb."""
    device.init(0)
    options = options or default_options(case)
    tiles, jobs, n_parts = plan(case, options)
    if pool is None:
        pool = native_pool(case)
    dp = device.DevicePass(case.params, case.trees, tiles, jobs, n_parts, case.n_rows, case.blocks,
                           case.desc if with_desc else None, case.pos, pool_blocks=case.n_blocks, static=static,
                           rows_in_pool=rows_in_pool)
    Q, Kb, Vb = dev_u16(case.Q), dev_u16(case.Kb), dev_u16(case.Vb)
    O = torch.zeros_like(Q)
    if rows_in_pool:
        append_rows(case, pool)
        Kb = Vb = None
    dp.run(Q, Kb, Vb, pool, O, merge=not two_step)
    if two_step:
        dp.merge(O)
    torch.cuda.synchronize()
    return to_host_u16(O).reshape(case.n_rows, -1)
