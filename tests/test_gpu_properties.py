"""The benchmark shapes at FULL size on the GPU, checked through size-independent
properties (the CPU checker cannot run them whole in seconds): split-count
invariance, page-permutation bit-invariance, V == 1, linearity in V, chunked
prefill == one pass, window >= context == global, plus float64 brute force on
sampled rows / sequences gathered back from the device pool.
"""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, host, synth
from oracle import binding as ob

from helpers import TOL, beyond_rounding

pytestmark = pytest.mark.gpu


def _workload(name, **kw):
    import bench
    device.init(0)
    return bench.make_workload(name, **kw)


def _run(w, dp=None, Q=None, Kb=None, Vb=None, pool=None):
    O = torch.zeros_like(w.Q)
    (dp or w.passes[0]).run(w.Q if Q is None else Q, w.Kb if Kb is None else Kb, w.Vb if Vb is None else Vb,
                            w.pool if pool is None else pool, O)
    torch.cuda.synchronize()
    return O


def _f32(t):
    return t.float().cpu().numpy()


def _gather(w, seq, table):
    """K, V float64 [P][Hkv][HD] of one sequence of workload w through esp_kv_gather."""
    p = w.params
    t = w.trees[seq]
    P = int(t["P"])
    kvw = p.Hkv * p.head_dim
    K = torch.zeros(P * kvw, dtype=torch.int16, device="cuda")
    V = torch.zeros_like(K)
    device.kv_gather(p, w.pool, table[int(t["table"]):], P, K, V)
    torch.cuda.synchronize()
    conv = lambda x: ob.to_f32(x.cpu().numpy().view(np.uint16), p.dtype).astype(np.float64).reshape(P, p.Hkv, p.head_dim)  # noqa: E731
    return conv(K), conv(V)


def _brute_rows(w, seq, rows, K, V, window=0):
    """float64 attention of the given rows (relative) of one sequence: cached keys + causal batch keys."""
    p = w.params
    t = w.trees[seq]
    base, P = int(t["base"]), int(t["P"])
    G = p.H // p.Hkv
    q = _f32(w.Q[base:base + int(t["M"])]).astype(np.float64).reshape(-1, p.H, p.head_dim)
    kb = _f32(w.Kb[base:base + int(t["M"])]).astype(np.float64).reshape(-1, p.Hkv, p.head_dim)
    vb = _f32(w.Vb[base:base + int(t["M"])]).astype(np.float64).reshape(-1, p.Hkv, p.head_dim)
    out = np.zeros((len(rows), p.H, p.head_dim))
    for i, r in enumerate(rows):
        Kall = np.concatenate([K, kb[:r + 1]])
        Vall = np.concatenate([V, vb[:r + 1]])
        lo = max(0, P + r - window + 1) if window > 0 else 0
        for h in range(p.H):
            s = Kall[lo:, h // G] @ q[r, h] * float(p.scale)
            e = np.exp(s - s.max())
            out[i, h] = (e / e.sum()) @ Vall[lo:, h // G]
    return out.reshape(len(rows), -1)


# ---------------------------------------------------------------- batched decode, full size
def test_c2_full_size_parity_on_sampled_sequences_and_invariances():
    w = _workload("c2_batched_decode")
    p = w.params
    O = _f32(_run(w))
    # float64 brute force on three whole sequences (shortest, longest, one other)
    lens = [P for P, _ in w.seqs]
    for seq in {int(np.argmin(lens)), int(np.argmax(lens)), 7}:
        K, V = _gather(w, seq, w.passes[0].blocks)
        want = _brute_rows(w, seq, [0], K, V)
        b = int(w.trees[seq]["base"])
        assert np.abs(O[b:b + 1] - want).max() <= 2e-3
    # split-count invariance: one workgroup per (sequence, head) ... far more than the device holds
    for wg in (64, 4096):
        opts = host.options_mi355x(1, wg)
        tiles, jobs, n_parts = host.plan_tiles(w.trees, p.Hkv, 0, None, opts)
        dp = device.DevicePass(p, w.trees, tiles, jobs, n_parts, w.n_rows, w.tables[0], None, None)
        assert np.abs(_f32(_run(w, dp)) - O).max() <= 1e-3
    # the reference planner's own records (8-row tiles, 256-threadgroup budget)
    opts = host.options_reference()
    p.rows_per_tile = opts.rows_per_tile
    tiles, jobs, n_parts = host.plan_tiles(w.trees, device.plan_hint(p)[1], 0, None, opts)
    dp = device.DevicePass(p, w.trees, tiles, jobs, n_parts, w.n_rows, w.tables[0], None, None)
    assert np.abs(_f32(_run(w, dp)) - O).max() <= 1e-3
    p.rows_per_tile = 1


def test_c2_page_permutation_is_bit_invariant_at_full_size():
    """Move every page of one table to a fresh place in the pool: same bits out."""
    w = _workload("c2_batched_decode")
    p = w.params
    O1 = _run(w)
    page = 2 * p.bt * p.Hkv * p.head_dim
    src = torch.from_numpy(w.tables[0].astype(np.int64)).cuda()
    dst_ids = w.tables[1][:len(w.tables[0])]          # pages of another rotation set: disjoint from set 0
    dst = torch.from_numpy(dst_ids.astype(np.int64)).cuda()
    pool2 = w.pool.clone().view(-1, page)
    pool2[dst] = w.pool.view(-1, page)[src]
    dp = device.DevicePass(p, w.trees, w.tiles, w.jobs, w.n_parts, w.n_rows, dst_ids, None, None)
    O2 = _run(w, dp, pool=pool2.view(-1))
    assert torch.equal(O1.view(torch.int16), O2.view(torch.int16))


# ---------------------------------------------------------------- verify at 32K, full size
def test_c5_full_size_v_one_linearity_and_row0_equals_decode():
    w = _workload("c5_verify")
    p = w.params
    O = _f32(_run(w))
    # V == 1 (cache and batch)  =>  O == 1
    O1 = _f32(_run(w, Vb=torch.ones_like(w.Vb), pool=_pool_with_v(w, 1.0)))
    assert np.abs(O1 - 1.0).max() <= 2e-3
    # linearity in V: O(V) - O(V') depends on V - V' only through the same softmax weights;
    # with V' = 2 V the output doubles
    O2 = _f32(_run(w, Vb=w.Vb * 2, pool=_pool_with_v(w, None, scale=2.0)))
    assert np.abs(O2 - 2 * O).max() <= 2 * TOL   # two results, each within the bar
    # row 0 of every verify tree sees the cache + itself: equal to a decode pass of that row
    trees = w.trees.copy()
    trees["M"] = 1
    pd = synth.make_params(p.H, p.Hkv, p.head_dim, p.dtype, p.bt, rows_per_tile=1)
    resident, groups = device.plan_hint(pd)
    tiles, jobs, n_parts = host.plan_tiles(trees, groups, 0, None, host.options_mi355x(1, resident))
    dp = device.DevicePass(pd, trees, tiles, jobs, n_parts, w.n_rows, w.tables[0], None, None)
    Od = _f32(_run(w, dp))
    for t in w.trees:
        b = int(t["base"])
        assert np.abs(Od[b] - O[b]).max() <= 1e-3
    # float64 brute force on one sequence, all 4 rows (verify chain == causal among the drafts)
    K, V = _gather(w, 3, w.passes[0].blocks)
    want = _brute_rows(w, 3, [0, 1, 2, 3], K, V)
    b = int(w.trees[3]["base"])
    assert np.abs(O[b:b + 4] - want).max() <= 2e-3


def _pool_with_v(w, value, scale=None):
    """A copy of the pool whose V planes are `value` (or scaled): native layout, K plane then V plane per (block, head)."""
    p = w.params
    plane = p.bt * p.head_dim
    pv = w.pool.clone().view(-1, 2, plane)
    if value is not None:
        pv[:, 1] = value
    else:
        pv[:, 1] *= scale
    return pv.view(-1)


# ---------------------------------------------------------------- chunked prefill, full size
def test_c3_chunked_prefill_equals_one_pass_and_brute_force_rows():
    """8192 tokens: 4 chunks of 2048 against the growing paged cache (kv_save between chunks)
    == one 8192-row causal pass, row by row; sampled rows against float64."""
    device.init(0)
    H, Hkv, HD, bt, N = 40, 8, 128, 16, 8192
    p = synth.make_params(H, Hkv, HD, abi.ESP_BF16, bt, rows_per_tile=128)
    p.rows_per_tile = device.plan_hint3(p)[2]
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    mk = lambda *s: (torch.randn(*s, generator=g, device="cuda") * 0.5).to(torch.bfloat16)  # noqa: E731
    Q, Kb, Vb = mk(N, H * HD), mk(N, Hkv * HD), mk(N, Hkv * HD)
    n_blocks = 1024
    pool = torch.zeros(n_blocks * 2 * bt * Hkv * HD, dtype=torch.bfloat16, device="cuda")
    table = np.random.default_rng(3).permutation(n_blocks).astype(np.int32)[:N // bt]
    resident, groups = device.plan_hint(p)

    def run(trees, O):
        tiles, jobs, n_parts = host.plan_tiles(trees, groups, 0, None, host.options_mi355x(p.rows_per_tile, resident))
        dp = device.DevicePass(p, trees, tiles, jobs, n_parts, N, table, None, None)
        dp.run(Q, Kb, Vb, pool, O)

    whole = torch.zeros_like(Q)
    run(np.array([(0, 0, 0, N)], abi.TREE_DT), whole)
    torch.cuda.synchronize()
    chunked = torch.zeros_like(Q)
    for s in range(0, N, 2048):
        run(np.array([(s, s, 0, 2048)], abi.TREE_DT), chunked)
        saves = np.zeros(2048, abi.KVSAVE_DT)
        pos = s + np.arange(2048)
        saves["src_row"], saves["block"], saves["pos"] = pos, table[pos // bt], pos % bt
        device.kv_save(p, Kb, Vb, pool, device.to_dev(saves), len(saves))
    torch.cuda.synchronize()
    a, b = _f32(whole), _f32(chunked)
    assert beyond_rounding(a, b, abi.ESP_BF16, True) <= 2e-3   # two bf16 results: one unit in the last place of the stored output is taken off first
    # sampled rows against float64 (K / V of the whole sequence are the batch rows themselves)
    q = _f32(Q).astype(np.float64).reshape(N, H, HD)
    k = _f32(Kb).astype(np.float64).reshape(N, Hkv, HD)
    v = _f32(Vb).astype(np.float64).reshape(N, Hkv, HD)
    for r in (0, 1, 127, 128, 2047, 2048, 5000, 8191):
        for h in (0, 7, 39):
            s_ = k[:r + 1, h // 5] @ q[r, h] * float(p.scale)
            e = np.exp(s_ - s_.max())
            want = (e / e.sum()) @ v[:r + 1, h // 5]
            assert beyond_rounding(b[r, h * HD:(h + 1) * HD], want, abi.ESP_BF16, False) <= TOL, (r, h)
    # what esp_kv_save wrote is what esp_kv_gather returns: bit exact
    Kg = torch.zeros(N * Hkv * HD, dtype=torch.bfloat16, device="cuda")
    Vg = torch.zeros_like(Kg)
    device.kv_gather(p, pool, device.to_dev(table), N, Kg, Vg)
    torch.cuda.synchronize()
    assert torch.equal(Kg.view(torch.int16), Kb.reshape(-1).view(torch.int16))
    assert torch.equal(Vg.view(torch.int16), Vb.reshape(-1).view(torch.int16))


# ---------------------------------------------------------------- sliding window + global, full size
def test_c4_decode_window_properties_at_full_size():
    ws = _workload("c4_decode_sliding")
    wg = _workload("c4_decode_global")
    Os, Og = _f32(_run(ws)), _f32(_run(wg))
    assert np.abs(Os - Og).max() > 1e-3                      # the window really hides keys
    # window >= context + 1  ==  global, on the same pool and tables
    p = ws.params
    p.window = 16384 + 1
    tiles, jobs, n_parts = host.plan_tiles(ws.trees, p.Hkv, p.window, ws.pos, host.options_mi355x(1, device.plan_hint(p)[0]))
    dp = device.DevicePass(p, ws.trees, tiles, jobs, n_parts, ws.n_rows, ws.tables[0], None, ws.pos)
    Ow = _f32(_run(ws, dp))
    p.window = 1024
    assert np.abs(Ow - Og).max() <= 1e-3
    # float64 brute force on two sequences, both layer kinds
    for w, O, win in ((ws, Os, 1024), (wg, Og, 0)):
        for seq in (0, 5):
            K, V = _gather(w, seq, w.passes[0].blocks)
            want = _brute_rows(w, seq, [0], K, V, window=win)
            b = int(w.trees[seq]["base"])
            assert np.abs(O[b:b + 1] - want).max() <= 2e-3


def test_c4_prefill_sliding_and_global_sampled_rows():
    for name, win in (("c4_prefill_sliding", 1024), ("c4_prefill_global", 0)):
        w = _workload(name)
        O = _f32(_run(w))
        K, V = _gather(w, 2, w.passes[0].blocks)
        rows = [0, 1, 500, 1023]
        want = _brute_rows(w, 2, rows, K, V, window=win)
        b = int(w.trees[2]["base"])
        got = np.stack([O[b + r] for r in rows])
        assert np.abs(got - want).max() <= 2e-3, name


# ---------------------------------------------------------------- head dim 512 (Gemma 4 global layers), full size
def test_g4_global512_decode_and_prefill_at_full_size():
    """Float64 brute force on sampled sequences / rows, split-count invariance of the decode, and row 0 of
    a prefill chunk == the decode step on the same cache (the tiled and the streaming kernel agree)."""
    wd = _workload("g4_global512_decode")
    Od = _f32(_run(wd))
    for seq in (0, 6):
        K, V = _gather(wd, seq, wd.passes[0].blocks)
        want = _brute_rows(wd, seq, [0], K, V)
        b = int(wd.trees[seq]["base"])
        assert np.abs(Od[b:b + 1] - want).max() <= 2e-3
    p = wd.params
    for wgs in (64, 2048):
        tiles, jobs, n_parts = host.plan_tiles(wd.trees, p.Hkv, 0, None, host.options_mi355x(1, wgs))
        dp = device.DevicePass(p, wd.trees, tiles, jobs, n_parts, wd.n_rows, wd.tables[0], None, None)
        assert np.abs(_f32(_run(wd, dp)) - Od).max() <= 1e-3
    del wd
    wp = _workload("g4_global512_prefill")
    Op = _f32(_run(wp))
    K, V = _gather(wp, 3, wp.passes[0].blocks)
    rows = [0, 1, 63, 64, 700, 1023]
    want = _brute_rows(wp, 3, rows, K, V)
    b = int(wp.trees[3]["base"])
    assert np.abs(np.stack([Op[b + r] for r in rows]) - want).max() <= 2e-3
    # row 0 of sequence 3 as a one-row decode pass over the same pool and table
    pd = synth.make_params(p.H, p.Hkv, p.head_dim, p.dtype, p.bt, rows_per_tile=1)
    t = wp.trees[3]
    trees = np.array([(0, int(t["P"]), int(t["table"]), 1)], abi.TREE_DT)
    tiles, jobs, n_parts = host.plan_tiles(trees, pd.Hkv, 0, None, host.options_mi355x(1, device.plan_hint(pd)[0]))
    dp = device.DevicePass(pd, trees, tiles, jobs, n_parts, 1, wp.tables[0], None, None)
    O1 = torch.zeros_like(wp.Q[b:b + 1])
    dp.run(wp.Q[b:b + 1].contiguous(), wp.Kb[b:b + 1].contiguous(), wp.Vb[b:b + 1].contiguous(), wp.pool, O1)
    torch.cuda.synchronize()
    assert np.abs(_f32(O1) - Op[b:b + 1]).max() <= 1e-3


def test_c1_single_decode_matches_checker_exactly_sized():
    """The reference's own CPU-runnable shape: small enough for the checker to run whole."""
    from gpu_utils import run_case
    from helpers import max_abs, oracle_direct
    c = synth.c1_single_decode()
    got = run_case(c)
    assert max_abs(got, oracle_direct(c, threads=8), c.params.dtype) <= 2e-3
