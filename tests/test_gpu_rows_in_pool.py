"""A pass whose own rows are read from the pool: esp_attn_forward without Kb / Vb, after the rows were appended
(esp_kv_save, or esp_attn_prep with a row table and no Kb / Vb of its own). Held to the form with Kb / Vb bit for bit
(the same bytes reach the same arithmetic by another road) and to the CPU checker within the path's bar."""
import numpy as np
import pytest

from espetero_amd import abi, device, host, synth

from helpers import max_abs, oracle_direct, small_case, tol_for

pytestmark = pytest.mark.gpu


def pool_case(seed, seqs, **kw):
    """A case whose block lists (or rings) reach P + M: made with P + M cached keys per sequence, then told that only
    P of them are cached - what lies behind them in the pool is overwritten by the append."""
    c = small_case(seed=seed, seqs=tuple((P + M, M) for P, M in seqs), **kw)
    for t, (P, M) in zip(c.trees, seqs):
        t["P"] = P
        b = int(t["base"])
        c.pos[b:b + M, 0:3] = (P + np.arange(M))[:, None]
    c.meta["seqs"] = list(seqs)
    return c


def _both(case, options=None):
    from gpu_utils import run_case
    print(f"rows in pool: seqs={case.meta['seqs']} HD={case.params.head_dim} R={case.params.rows_per_tile} bt={case.params.bt} "
          f"window={case.params.window} ring={case.params.ring}", flush=True)
    want = run_case(case, options)
    got = run_case(case, options, rows_in_pool=True)
    assert (got == want).all(), "reading the rows from the pool changes the output"
    err = max_abs(got, oracle_direct(case, threads=8), case.params.dtype)
    assert err <= tol_for(case.params.dtype), err


@pytest.mark.parametrize("kw", [
    dict(seqs=((0, 200),)),                                                        # first chunk: nothing cached
    dict(seqs=((256, 300),), H=10, Hkv=2, dtype=abi.ESP_BF16),                     # a later chunk, GQA 5, bf16
    dict(seqs=((32, 40), (56, 77), (213, 1)), fill_unused=True),                   # three trees: P - base = 32, 16, 96
    dict(seqs=((1024, 140),), H=4, Hkv=2, HD=256),                                 # head dim 256, the mask-free runs
    dict(seqs=((96, 130),), H=4, Hkv=2, bt=64),                                    # the reference's block size
    dict(seqs=((512, 200),), H=4, Hkv=2, window=128),                              # sliding window over block lists
    dict(seqs=((128, 100),), H=4, Hkv=2, bidi=1, desc_fn=lambda M: synth.image_desc(M, 10, 90)),
    dict(seqs=((64, 150),), H=4, Hkv=2, HD=512, rows_per_tile=64),                 # head dim 512
    dict(seqs=((3008, 100),), H=4, Hkv=2, split=64),                               # split tiles: the last part owns the rows
    dict(seqs=((3008, 1400),), H=2, Hkv=1),                                        # 69 steps: the 64-step address window is refilled inside the pass's own rows
    dict(seqs=((2048, 2200),), H=2, Hkv=1, HD=256, bt=32),                         # the same at head dim 256 with 32-token blocks
    dict(seqs=((1024, 1200),), H=2, Hkv=1, HD=512, rows_per_tile=64, bt=64),       # 512: 64 sub-blocks at a time, 139 in all
    dict(seqs=((16, 400),), H=4, Hkv=2),                                           # a first step of 1 cached sub-block and 3 of the pass's own
    dict(seqs=((48, 300), (44, 140)), H=2, Hkv=1, HD=256, dtype=abi.ESP_BF16),     # 3 + 1, and (P - base = -256) 2 3/4 + 1 1/4, head dim 256
    dict(seqs=((32, 24), (40, 330)), H=4, Hkv=2, window=96, fill_unused=True),     # P - base = 16: the cached range ends inside a sub-block; under a window
])
def test_tiled_kernel_reads_its_rows_from_the_pool(kw):
    split = kw.pop("split", None)
    c = pool_case(61, **{"rows_per_tile": 128, **kw})
    _both(c, host.options_mi355x(c.params.rows_per_tile, split) if split else None)


@pytest.mark.parametrize("kw", [
    dict(seqs=((70, 1), (33, 1), (0, 1), (16, 1)), rows_per_tile=1),               # decode rows at any position of a page
    dict(seqs=((1030, 4), (90, 4)), rows_per_tile=4, desc_fn=lambda M: synth.verify_desc(M, 1)),   # a root and its chain
    dict(seqs=((777, 1), (100, 1)), H=4, Hkv=2, HD=256, rows_per_tile=1),
    dict(seqs=((300, 2),), H=8, Hkv=2, HD=512, rows_per_tile=2, dtype=abi.ESP_BF16),
    dict(seqs=((300, 4), (50, 4)), H=8, Hkv=1, HD=512, rows_per_tile=4, desc_fn=lambda M: synth.verify_desc(M, 1)),   # two wavefront pairs
    dict(seqs=((400, 6), (64, 2)), H=4, Hkv=2, rows_per_tile=8, bt=64),            # short causal chunks on the streaming kernel
    dict(seqs=((900, 1), (2000, 1)), window=256, ring_layer=True, rows_per_tile=1),  # rings: a decode row overwrites what no row sees
    dict(seqs=((5000, 1), (900, 1)), H=32, Hkv=4, rows_per_tile=1, split=256),     # split ranges: the last part owns the row
])
def test_stream_kernel_reads_its_rows_from_the_pool(kw):
    split = kw.pop("split", None)
    c = pool_case(62, **kw)
    _both(c, host.options_mi355x(c.params.rows_per_tile, split) if split else None)


def test_prep_appends_without_kb_vb_and_the_attention_reads_the_rows_there():
    """esp_attn_prep with a row table and no Kb / Vb, then esp_attn_forward without Kb / Vb: O and the pool are those of
    prep (with Kb / Vb) + attention + esp_kv_save, bit for bit; O is the checker's within the bar."""
    import torch
    from gpu_utils import dev_u16, to_host_u16
    from oracle import binding as ob
    device.init(0)
    H, Hkv, HD, bt, dtype, P, M = 10, 2, 128, 16, abi.ESP_BF16, 256, 300
    pp, a = synth.make_prep("omni", H, Hkv, HD, dtype, M, seed=9, bt=bt)
    a["pos"][:, :3] = (P + np.arange(M))[:, None]
    c = pool_case(63, ((P, M),), H=H, Hkv=Hkv, HD=HD, dtype=dtype, bt=bt, rows_per_tile=128)
    ap = c.params
    ap.scale = 1.0                                        # the omni prep scales the queries itself
    table = np.full((M, 4), -1, np.int32)
    q = P + np.arange(M)
    table[:, 0], table[:, 1] = c.blocks[q // bt], q % bt
    dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
    X, qn, kn, pos, invf, sel = dev(a["X"]), dev(a["qn_w"]), dev(a["kn_w"]), dev(a["pos"]), dev(a["inv_freq"]), dev(a["rope_sel"])
    from gpu_utils import native_pool, plan
    tiles, jobs, n_parts = plan(c, host.options_mi355x(128, 64))
    outs, pools = [], []
    for in_pool in (False, True):
        pool = native_pool(c)
        Q = torch.zeros(M, ap.q_ld, dtype=torch.int16, device="cuda")
        Kb = None if in_pool else torch.zeros(M, ap.kv_ld, dtype=torch.int16, device="cuda")
        Vb = None if in_pool else torch.zeros_like(Kb)
        O = torch.zeros_like(Q)
        dp = device.DevicePass(ap, c.trees, tiles, jobs, n_parts, M, c.blocks, None, None, pool_blocks=c.n_blocks, rows_in_pool=in_pool)
        if in_pool:
            device.attn_prep(pp, X, qn, kn, pos, invf, sel, Q, None, None, dev(table), pool, M)
            dp.run(Q, None, None, pool, O)
        else:
            device.attn_prep(pp, X, qn, kn, pos, invf, sel, Q, Kb, Vb, None, None, M)
            dp.run(Q, Kb, Vb, pool, O)
            e = np.zeros(M, abi.KVSAVE_DT)
            e["src_row"], e["block"], e["pos"] = np.arange(M), table[:, 0], table[:, 1]
            device.kv_save(ap, Kb, Vb, pool, device.to_dev(e), M)
        torch.cuda.synchronize()
        outs.append(to_host_u16(O).reshape(M, -1))
        pools.append(to_host_u16(pool))
    assert (outs[0] == outs[1]).all() and (pools[0] == pools[1]).all()
    qh, kb, vb = ob.attn_prep(pp, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], M)
    want = ob.attn_direct(ap, qh, kb, vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees, n_threads=8)
    assert max_abs(outs[1], want, dtype) <= tol_for(dtype)
