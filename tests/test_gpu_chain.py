"""A decode chain kept on the device: prep (with the folded append) -> attention -> esp_chain_advance,
K steps enqueued back to back and captured in a HIP graph, against the CPU checker driven step by step
from the host (the reference's statement about its own chains: "tokens are identical to step-by-step
decoding", docs/design.md:232)."""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, host, synth
from oracle import binding as ob

pytestmark = pytest.mark.gpu

K = 10
P0 = [70, 33, 500, 1030, 16, 0]
# (query heads, KV heads, head dim, tokens per block, prep arrangement): the benchmark's Qwen shape, a sliding-layer
# Gemma shape at the reference's block size, and Gemma 4's 512-dim heads (wavefront pairs, open-ended ranges)
SHAPES = [(8, 2, 128, 16, "omni"), (4, 2, 256, 64, "gemma"), (8, 1, 512, 16, "gemma")]
# (shape, window): 0 = a layer that keeps every key in listed blocks; > 0 = a sliding layer whose slot holds a ring of
# ceil(window / block) consecutive blocks, key j in block (j / block) % ring (80_gemma.metal:139), which the chain's
# appends overwrite as they go
CASES = [(s, 0) for s in SHAPES] + [((8, 2, 128, 16, "omni"), 100), ((4, 2, 256, 64, "gemma"), 128), ((16, 8, 256, 16, "gemma"), 48)]


def _slot_block(ap, blocks, table, j):
    """Physical block of key j of the slot whose record says `table` (arrays or scalars)."""
    bi = j // ap.bt
    return table + bi % ap.ring if ap.ring else blocks[table + bi]


def _setup(shape, window, seed=12):
    H, HKV, HD, BT, kind = shape
    rng = np.random.default_rng(seed)
    n = len(P0)
    ring = (window + BT - 1) // BT if window else 0
    ap = synth.make_params(H, HKV, HD, abi.ESP_F16, BT, window=window, ring=ring, rows_per_tile=1)
    pp, a = synth.make_prep(kind, H, HKV, HD, abi.ESP_F16, n, seed=seed, bt=BT)
    nb = [ring if ring else (p + K + BT) // BT for p in P0]    # room for the K tokens the chain appends
    n_blocks = sum(nb) + 3
    perm = rng.permutation(n_blocks).astype(np.int32)
    blocks = perm[:sum(nb)].copy()                             # a ring's blocks are not listed: its record names the first
    trees = np.zeros(n, abi.TREE_DT)
    kvw = HKV * HD
    pool = np.zeros(n_blocks * 2 * BT * kvw, np.uint16)       # reference layout
    pv = pool.reshape(n_blocks, 2, BT, kvw)
    off = 0
    for i, p in enumerate(P0):
        trees[i] = (i, p, off, 1)
        for j in range(max(0, p - ring * BT) if ring else 0, p):   # a ring holds the last ring * block keys
            b = _slot_block(ap, blocks, off, j)
            pv[b, 0, j % BT] = ob.from_f32(rng.standard_normal(kvw).astype(np.float32) * 0.5, ap.dtype)
            pv[b, 1, j % BT] = ob.from_f32(rng.standard_normal(kvw).astype(np.float32) * 0.5, ap.dtype)
        off += nb[i]
    X = (rng.standard_normal((K, n, pp.x_ld)).astype(np.float32) * 0.5)   # values as in the other tests: |v| < 4, half a unit in the last place of an output < 1e-3
    return ap, pp, a, trees, blocks, pool, n_blocks, X


def _host_chain(ap, trees, blocks, pool, Q, Kb, Vb):
    BT = ap.bt
    """The checker, one step at a time, every record rebuilt on the host. Q / Kb / Vb [K][n][...]: the
    prepared rows of every step (storage bits); each step's K / V row joins the cache after its attention."""
    n = len(trees)
    pool = pool.copy()
    trees = trees.copy()
    out = []
    for s in range(K):
        pos = np.zeros((n, 4), np.int32)
        pos[:, :3] = trees["P"][:, None]
        desc = np.zeros((n, 4), np.int32)
        out.append(ob.attn_direct(ap, Q[s], Kb[s], Vb[s], pool, blocks, desc, pos, trees, n_threads=4))
        e = np.zeros(n, abi.KVSAVE_DT)
        e["src_row"], e["block"], e["pos"] = np.arange(n), _slot_block(ap, blocks, trees["table"], trees["P"]), trees["P"] % BT
        ob.kv_save(ap, Kb[s], Vb[s], pool, e)
        trees["P"] += 1
    return np.stack(out), pool


@pytest.mark.parametrize("shape,window", CASES)
def test_device_chain_matches_the_checker_step_by_step_and_replays_identically(shape, window):
    device.init(0)
    ap, pp, a, trees, blocks, pool_ref, n_blocks, X = _setup(shape, window)
    n = len(trees)
    BT = ap.bt
    print(f"chain shape {shape} window {window} ring {ap.ring}", flush=True)

    dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
    ref = dev(pool_ref.view(np.int16))
    pool0 = torch.empty_like(ref)
    device.kv_relayout(ap, ref, abi.ESP_LAYOUT_REFERENCE, pool0, abi.ESP_LAYOUT_NATIVE, n_blocks)
    resident, groups = device.plan_hint(ap)
    pos0 = np.zeros((n, 4), np.int32)
    pos0[:, :3] = trees["P"][:, None]
    tiles, jobs, n_parts = host.plan_tiles(trees, groups, window, pos0 if window else None, host.options_mi355x(1, resident))
    tiles = host.open_ended(tiles, trees)
    assert (tiles["k1"] == 2**31 - 1).sum() == n               # one open range per sequence
    table0 = np.full((n, 4), -1, np.int32)
    table0[:, 0] = _slot_block(ap, blocks, trees["table"], trees["P"])
    table0[:, 1] = trees["P"] % BT
    # device-resident state of the chain, and its initial values to go back to before every run
    init = dict(trees=device.to_dev(trees), pos=dev(pos0), table=dev(table0), pool=pool0)
    st = {k: v.clone() for k, v in init.items()}
    blocks_d = dev(blocks)
    dp = device.DevicePass(ap, trees, tiles, jobs, n_parts, n, blocks, None, None)
    dp.trees = st["trees"]                                      # the pass reads the records the chain advances
    if window:
        dp.pos = st["pos"]                                      # and, for the window rule, the positions it advances
    Xd, qn, kn = dev(X), dev(a["qn_w"]), dev(a["kn_w"])
    inv_freq, sel = dev(a["inv_freq"]), dev(a["rope_sel"])
    Q = torch.zeros(K, n, ap.q_ld, dtype=torch.float16, device="cuda")      # every step's prepared rows are kept
    Kb = torch.zeros(K, n, ap.kv_ld, dtype=torch.float16, device="cuda")
    Vb = torch.zeros_like(Kb)
    O = torch.zeros(K, n, ap.q_ld, dtype=torch.float16, device="cuda")

    def chain():
        for s in range(K):
            device.attn_prep(pp, Xd[s], qn, kn, st["pos"], inv_freq, sel, Q[s], Kb[s], Vb[s], st["table"], st["pool"], n)
            dp.run(Q[s], Kb[s], Vb[s], st["pool"], O[s])
            device.chain_advance(st["trees"], n, st["pos"], st["table"], blocks_d, BT, ap.ring)

    def reset():
        for k in st:
            st[k].copy_(init[k])
        O.zero_()

    bits = lambda t: t.view(torch.int16).cpu().numpy().view(np.uint16)  # noqa: E731
    ref_out = {}

    def check(tag):
        torch.cuda.synchronize()
        if not ref_out:   # the checker runs on the rows the device prepared, so that this compares attention with attention
            ref_out["want"], ref_out["pool"] = _host_chain(ap, trees, blocks, pool_ref, bits(Q), bits(Kb), bits(Vb))
        want = ref_out["want"]
        got = ob.to_f32(bits(O), ap.dtype)
        err = float(np.abs(got - ob.to_f32(want, ap.dtype)).max())
        print(f"chain {tag}: max abs err {err:.2e}", flush=True)
        assert err <= 2e-3, (tag, err)
        # the records ended where K steps of host bookkeeping end
        t = st["trees"].cpu().numpy().view(abi.TREE_DT)
        assert (t["P"] == trees["P"] + K).all()
        assert (st["pos"].cpu().numpy()[:, 0] == trees["P"] + K).all()
        return O.clone()

    reset()
    chain()                                                     # enqueued eagerly, no host work in between
    eager = check("eager")
    # the prep inside the chain saw the positions the device advanced: its rows are the checker's rows for
    # host-built positions (to the prep kernel's bar of one unit in the last place)
    for s_ in range(K):
        pos = np.zeros((n, 4), np.int32)
        pos[:, :3] = (trees["P"] + s_)[:, None]
        qw, kw, vw = ob.attn_prep(pp, X[s_], a["qn_w"], a["kn_w"], pos, a["inv_freq"], a["rope_sel"], n)
        for g_, w_ in ((bits(Q[s_]), qw), (bits(Kb[s_]), kw), (bits(Vb[s_]), vw)):
            assert np.abs(ob.to_f32(g_, ap.dtype).astype(np.float64) - ob.to_f32(w_, ap.dtype)).max() <= 2.0 ** -8
    # every appended token is in the pool where host bookkeeping puts it: bit for bit
    back = torch.empty_like(ref)
    device.kv_relayout(ap, st["pool"], abi.ESP_LAYOUT_NATIVE, back, abi.ESP_LAYOUT_REFERENCE, n_blocks)
    torch.cuda.synchronize()
    assert np.array_equal(bits(back), ref_out["pool"])
    Kg = torch.zeros((max(P0) + K) * ap.kv_ld, dtype=torch.float16, device="cuda")
    Vg = torch.zeros_like(Kg)
    for i, p in enumerate(P0 if not ap.ring else []):           # listed blocks also read back in token order
        device.kv_gather(ap, st["pool"], blocks_d[int(trees[i]["table"]):], p + K, Kg, Vg)
        torch.cuda.synchronize()
        kw, vw = ob.kv_gather(ap, ref_out["pool"], blocks[int(trees[i]["table"]):], p + K)
        assert np.array_equal(bits(Kg)[:(p + K) * ap.kv_ld].reshape(p + K, -1), kw)
        assert np.array_equal(bits(Vg)[:(p + K) * ap.kv_ld].reshape(p + K, -1), vw)

    # the chain with attn_prep fused into the attention kernel (no prep dispatch, no Q / Kb / Vb in memory):
    # the outputs and every pool byte of the three-dispatch chain, bit for bit
    if ap.head_dim != 512:
        eager_pool = st["pool"].clone()
        reset()
        for s in range(K):
            device.decode_fused(pp, ap, Xd[s], qn, kn, st["pos"], inv_freq, sel, st["table"], st["pool"], dp, O[s])
            device.chain_advance(st["trees"], n, st["pos"], st["table"], blocks_d, BT, ap.ring)
        torch.cuda.synchronize()
        assert torch.equal(O.view(torch.int16), eager.view(torch.int16)), "fused decode differs from prep + attention"
        assert torch.equal(st["pool"].view(torch.int16), eager_pool.view(torch.int16)), "fused decode appended other bytes"
        print("chain fused: identical outputs and pool", flush=True)

    # the same chain as one HIP graph, replayed with eager work and synchronisations in between
    reset()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            chain()
    torch.cuda.synchronize()
    for rep in range(3):
        reset()
        torch.cuda.synchronize()
        g.replay()
        got = check(f"graph replay {rep}")
        assert torch.equal(got.view(torch.int16), eager.view(torch.int16))


@pytest.mark.parametrize("H,Hkv,HD,kind,dtype", [(8, 2, 128, "omni", abi.ESP_F16), (16, 2, 128, "qwen35x", abi.ESP_BF16),
                                                 (4, 2, 256, "gemma", abi.ESP_F16), (8, 2, 256, "qwen35", abi.ESP_BF16)])
def test_fused_prep_on_verify_trees_is_prep_then_attention_bit_for_bit(H, Hkv, HD, kind, dtype):
    """Short verify trees (a root row and a chain of three drafts, 4 rows = one tile) and plain decode rows in one
    pass: esp_attn_decode_fused against esp_attn_prep followed by esp_attn_forward, with the folded append, split
    ranges and the merge. Outputs and pool bytes must be identical; the first is also held to the checker."""
    kind = kind.rstrip("x")
    device.init(0)
    rng = np.random.default_rng(23)
    BT = 16
    seqs = [(700, 4), (33, 4), (2000, 1), (0, 3)]
    n_rows = sum(m for _, m in seqs)
    ap = synth.make_params(H, Hkv, HD, dtype, BT, rows_per_tile=4)
    pp, a = synth.make_prep(kind, H, Hkv, HD, dtype, n_rows, seed=29, bt=BT)
    nb = [(p + m + BT - 1) // BT for p, m in seqs]
    n_blocks = sum(nb) + 2
    perm = rng.permutation(n_blocks).astype(np.int32)
    blocks = perm[:sum(nb)].copy()
    trees = np.zeros(len(seqs), abi.TREE_DT)
    desc = np.zeros((n_rows, 4), np.int32)
    pos = np.zeros((n_rows, 4), np.int32)
    table = np.full((n_rows, 4), -1, np.int32)
    base = off = 0
    for i, (p, m) in enumerate(seqs):
        trees[i] = (base, p, off, m)
        if m > 1:
            desc[base:base + m] = synth.verify_desc(m, 1)
        pos[base:base + m, :3] = (p + np.arange(m))[:, None]
        tok = p + np.arange(m)
        table[base:base + m, 0] = blocks[off + tok // BT]
        table[base:base + m, 1] = tok % BT
        base += m
        off += nb[i]
    tdt = torch.float16 if dtype == abi.ESP_F16 else torch.bfloat16
    pool0 = (torch.randn(n_blocks * 2 * BT * ap.kv_ld, device="cuda") * 0.5).to(tdt)
    resident, groups = device.plan_hint(ap)
    tiles, jobs, n_parts = host.plan_tiles(trees, groups, 0, None, host.options_mi355x(4, 64))
    assert n_parts > 0
    dp = device.DevicePass(ap, trees, tiles, jobs, n_parts, n_rows, blocks, desc, pos, pool_blocks=n_blocks, fused=True)
    dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
    Xd, qn, kn, posd = dev(a["X"]), dev(a["qn_w"]), dev(a["kn_w"]), dev(pos)
    inv_freq, sel, tabd = dev(a["inv_freq"]), dev(a["rope_sel"]), dev(table)
    if kind == "qwen35":   # the sigmoid gate beside each query in the projection itself (40_attention.metal:47, :334-342)
        ap.gate = Xd.data_ptr()
        ap.gate_ld, ap.gate_hs, ap.gate_off = pp.x_ld, pp.q_hs, HD
    print(f"fused verify: H={H} Hkv={Hkv} HD={HD} {kind} tiles={len(tiles)} parts={n_parts}", flush=True)
    outs, pools = [], []
    for fused in (False, True):
        pool = pool0.clone()
        O = torch.zeros(n_rows, ap.q_ld, dtype=tdt, device="cuda")
        if fused:
            device.decode_fused(pp, ap, Xd, qn, kn, posd, inv_freq, sel, tabd, pool, dp, O)
        else:
            Q = torch.zeros(n_rows, ap.q_ld, dtype=tdt, device="cuda")
            Kb = torch.zeros(n_rows, ap.kv_ld, dtype=tdt, device="cuda")
            Vb = torch.zeros_like(Kb)
            device.attn_prep(pp, Xd, qn, kn, posd, inv_freq, sel, Q, Kb, Vb, tabd, pool, n_rows)
            dp.run(Q, Kb, Vb, pool, O)
        torch.cuda.synchronize()
        outs.append(O)
        pools.append(pool)
    assert bool(outs[0].any())
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16)), "fused output differs"
    assert torch.equal(pools[0].view(torch.int16), pools[1].view(torch.int16)), "fused append differs"
    assert not torch.equal(pools[0].view(torch.int16), pool0.view(torch.int16))
    ap.gate = None


def test_fused_decode_on_seeded_random_shapes_is_prep_then_attention_bit_for_bit():
    """40 seeded random decode / short-verify passes (head dim, grouping, element type, block size, prep arrangement,
    rows per tile, ragged cached lengths incl. empty ones, window over block lists, split target): the fused call and
    the two calls must leave identical outputs and identical pools."""
    device.init(0)
    rng = np.random.default_rng(77)
    dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
    for it in range(40):
        HD = int(rng.choice([128, 256]))
        G = int(rng.choice([1, 2, 4, 5, 8]))
        Hkv = int(rng.choice([1, 2, 4]))
        H = G * Hkv
        max_cols = 32 if HD == 128 else 16
        R = int(rng.integers(1, min(4, max_cols // G) + 1))
        BT = int(rng.choice([16, 32, 64]))
        dtype = int(rng.choice([abi.ESP_F16, abi.ESP_BF16]))
        kind = str(rng.choice(["omni", "gemma", "qwen35"]))
        window = int(rng.choice([0, 0, 200]))
        seqs = [(int(rng.choice([0, 1, 15, 16, 17, 300, 1500, 4000])), int(rng.integers(1, R + 1))) for _ in range(int(rng.integers(1, 7)))]
        n_rows = sum(m for _, m in seqs)
        ap = synth.make_params(H, Hkv, HD, dtype, BT, window=window, rows_per_tile=R)
        pp, a = synth.make_prep(kind, H, Hkv, HD, dtype, n_rows, seed=1000 + it, bt=BT)
        nb = [(p + m + BT - 1) // BT for p, m in seqs]
        n_blocks = sum(nb) + 2
        blocks = rng.permutation(n_blocks).astype(np.int32)[:sum(nb)].copy()
        trees = np.zeros(len(seqs), abi.TREE_DT)
        desc = np.zeros((n_rows, 4), np.int32)
        pos = np.zeros((n_rows, 4), np.int32)
        table = np.full((n_rows, 4), -1, np.int32)
        base = off = 0
        for i, (p, m) in enumerate(seqs):
            trees[i] = (base, p, off, m)
            if m > 1:
                desc[base:base + m] = synth.verify_desc(m, 1)
            tok = p + np.arange(m)
            pos[base:base + m, :3] = tok[:, None]
            table[base:base + m, 0] = blocks[off + tok // BT]
            table[base:base + m, 1] = tok % BT
            base += m
            off += nb[i]
        tdt = torch.float16 if dtype == abi.ESP_F16 else torch.bfloat16
        pool0 = (torch.randn(n_blocks * 2 * BT * ap.kv_ld, device="cuda") * 0.5).to(tdt)
        resident, groups = device.plan_hint(ap)
        tiles, jobs, n_parts = host.plan_tiles(trees, groups, window, pos if window else None, host.options_mi355x(R, int(rng.choice([8, 64, resident]))))
        print(f"fused random {it}: H={H} Hkv={Hkv} HD={HD} R={R} bt={BT} dtype={dtype} {kind} window={window} seqs={seqs} tiles={len(tiles)} parts={n_parts}", flush=True)
        dp = device.DevicePass(ap, trees, tiles, jobs, n_parts, n_rows, blocks, desc, pos, pool_blocks=n_blocks, fused=True)
        Xd, qn, kn, posd = dev(a["X"]), dev(a["qn_w"]), dev(a["kn_w"]), dev(pos)
        inv_freq, sel, tabd = dev(a["inv_freq"]), dev(a["rope_sel"]), dev(table)
        res = []
        for fused in (False, True):
            pool = pool0.clone()
            O = torch.zeros(n_rows, ap.q_ld, dtype=tdt, device="cuda")
            if fused:
                device.decode_fused(pp, ap, Xd, qn, kn, posd, inv_freq, sel, tabd, pool, dp, O)
            else:
                Q = torch.zeros(n_rows, ap.q_ld, dtype=tdt, device="cuda")
                Kb = torch.zeros(n_rows, ap.kv_ld, dtype=tdt, device="cuda")
                Vb = torch.zeros_like(Kb)
                device.attn_prep(pp, Xd, qn, kn, posd, inv_freq, sel, Q, Kb, Vb, tabd, pool, n_rows)
                dp.run(Q, Kb, Vb, pool, O)
            torch.cuda.synchronize()
            res.append((O, pool))
        assert torch.equal(res[0][0].view(torch.int16), res[1][0].view(torch.int16)), (it, "output")
        assert torch.equal(res[0][1].view(torch.int16), res[1][1].view(torch.int16)), (it, "pool")


def test_fused_decode_without_an_append_and_without_descriptors_leaves_the_pool_alone():
    """row_table NULL: the rows' K / V take part in the attention but are not written anywhere; desc NULL: plain decode
    rows. Outputs equal those of esp_attn_prep (no table) + esp_attn_forward, and the pool is untouched."""
    device.init(0)
    rng = np.random.default_rng(5)
    H, Hkv, HD, BT, dtype = 8, 2, 128, 16, abi.ESP_BF16
    seqs = [(900, 1), (31, 1), (0, 1)]
    n_rows = len(seqs)
    ap = synth.make_params(H, Hkv, HD, dtype, BT, rows_per_tile=1)
    pp, a = synth.make_prep("gemma", H, Hkv, HD, dtype, n_rows, seed=3, bt=BT)
    nb = [(p + BT - 1) // BT for p, _ in seqs]
    n_blocks = sum(nb) + 1
    blocks = rng.permutation(n_blocks).astype(np.int32)[:max(sum(nb), 1)].copy()
    trees = np.zeros(n_rows, abi.TREE_DT)
    pos = np.zeros((n_rows, 4), np.int32)
    off = 0
    for i, (p, m) in enumerate(seqs):
        trees[i] = (i, p, off, 1)
        pos[i, :3] = p
        off += nb[i]
    pool0 = (torch.randn(n_blocks * 2 * BT * ap.kv_ld, device="cuda") * 0.5).to(torch.bfloat16)
    resident, groups = device.plan_hint(ap)
    tiles, jobs, n_parts = host.plan_tiles(trees, groups, 0, None, host.options_mi355x(1, 32))
    dp = device.DevicePass(ap, trees, tiles, jobs, n_parts, n_rows, blocks, None, None, pool_blocks=n_blocks, fused=True)
    dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
    Xd, qn, kn, posd, inv_freq = dev(a["X"]), dev(a["qn_w"]), dev(a["kn_w"]), dev(pos), dev(a["inv_freq"])
    pool = pool0.clone()
    O1 = torch.zeros(n_rows, ap.q_ld, dtype=torch.bfloat16, device="cuda")
    device.decode_fused(pp, ap, Xd, qn, kn, posd, inv_freq, None, None, pool, dp, O1)
    torch.cuda.synchronize()
    assert torch.equal(pool.view(torch.int16), pool0.view(torch.int16))
    Q = torch.zeros(n_rows, ap.q_ld, dtype=torch.bfloat16, device="cuda")
    Kb = torch.zeros(n_rows, ap.kv_ld, dtype=torch.bfloat16, device="cuda")
    Vb = torch.zeros_like(Kb)
    O2 = torch.zeros_like(O1)
    device.attn_prep(pp, Xd, qn, kn, posd, inv_freq, None, Q, Kb, Vb, None, None, n_rows)
    dp.run(Q, Kb, Vb, pool, O2)
    torch.cuda.synchronize()
    assert bool(O1.any()) and torch.equal(O1.view(torch.int16), O2.view(torch.int16))
