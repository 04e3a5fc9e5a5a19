"""Host engine (C++ planner, KV pool, pass builder) against the integer
restatement of the reference's formulas in oracle/host_oracle.py, plus the
properties those formulas must keep. Integer work: every comparison is exact.
"""
import numpy as np
import pytest

from espetero_amd import abi, host
from oracle import host_oracle as ho


def _trees(rng, n, max_p=9000, max_m=1):
    out, base = [], 0
    for _ in range(n):
        P = int(rng.integers(0, max_p))
        M = int(rng.integers(1, max_m + 1))
        out.append((base, P, int(rng.integers(0, 100)), M))
        base += M
    return out


def _as_tuples(recs):
    return [tuple(int(x) for x in r) for r in recs]


# ---------------------------------------------------------------- planner, reference rule
@pytest.mark.parametrize("seed", range(12))
def test_reference_rule_is_bit_identical_to_plan_tiles(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, 20))
    trees = _trees(rng, n, max_m=int(rng.choice([1, 1, 4, 40, 300])))
    Hkv = int(rng.choice([1, 2, 4, 8]))
    split = int(rng.choice([0, 256, 512, 1024]))
    o = host.options_reference()
    o.split = split
    tiles, jobs, parts = host.plan_tiles(np.array(trees, abi.TREE_DT), Hkv, 0, None, o)
    wt, wj, wp = ho.plan_tiles(trees, Hkv, split)
    assert _as_tuples(tiles) == wt and _as_tuples(jobs) == wj and parts == wp
    # the windowless Gemma planner is the same rule (gemma.h:77-116 with window 0)
    gt, gj, gp, rows = ho.g4_plan_tiles(trees, Hkv, split, 0, None)
    assert rows == 8 and _as_tuples(tiles) == gt and _as_tuples(jobs) == gj and parts == gp


@pytest.mark.parametrize("seed", range(8))
def test_reference_rule_with_window_matches_g4_plan_tiles(seed):
    rng = np.random.default_rng(100 + seed)
    trees = _trees(rng, int(rng.integers(1, 10)), max_p=20000, max_m=int(rng.choice([1, 3, 30])))
    M = sum(t[3] for t in trees)
    pos = np.zeros((M, 4), np.int32)
    for base, P, _, m in trees:
        pos[base:base + m, 0] = P + np.arange(m)
    window = int(rng.choice([64, 1024, 4096]))
    o = host.options_reference()
    tiles, jobs, parts = host.plan_tiles(np.array(trees, abi.TREE_DT), 8, window, pos, o)
    wt, wj, wp, _ = ho.g4_plan_tiles(trees, 8, 512, window, pos.reshape(-1).tolist())
    assert _as_tuples(tiles) == wt and _as_tuples(jobs) == wj and parts == wp


def test_reference_rule_on_the_benchmark_shapes():
    """What the reference's planner does with its own constants on the benchmark shapes
    (256-threadgroup target, attn_split 512, 32-key granularity)."""
    o = host.options_reference()
    # single decode at 1024 keys, 4 KV heads: 32 tiles of 32 keys
    t, j, p = host.plan_tiles(np.array([(0, 1024, 0, 1)], abi.TREE_DT), 4, 0, None, o)
    assert len(t) == 32 and p == 32 and all(int(x["k1"] - x["k0"]) == 32 for x in t) and _as_tuples(j) == [(0, 1, 0, 32)]
    # 8 verify trees of 4 rows at 32K, 4 KV heads: 8 splits of 4096 keys each
    trees = [(4 * i, 32768, 2048 * i, 4) for i in range(8)]
    t, j, p = host.plan_tiles(np.array(trees, abi.TREE_DT), 4, 0, None, o)
    assert len(t) == 64 and p == 64 and all(int(x["k1"] - x["k0"]) == 4096 for x in t)
    assert all(int(x["nparts"]) == 8 and int(x["rows"]) == 4 for x in j)
    # one 2048-row prefill chunk, 8 KV heads: 256 unsplit 8-row tiles
    t, j, p = host.plan_tiles(np.array([(0, 4096, 0, 2048)], abi.TREE_DT), 8, 0, None, o)
    assert len(t) == 256 and p == 0 and len(j) == 0 and all(int(x["part"]) == -1 and int(x["last"]) == 1 for x in t)


# ---------------------------------------------------------------- planner, contractual algebra under any options
@pytest.mark.parametrize("seed", range(10))
def test_split_algebra_holds_for_both_rules(seed):
    rng = np.random.default_rng(200 + seed)
    trees = _trees(rng, int(rng.integers(1, 24)), max_p=40000, max_m=int(rng.choice([1, 4, 9])))
    M = sum(t[3] for t in trees)
    pos = np.zeros((M, 4), np.int32)
    for base, P, _, m in trees:
        pos[base:base + m, 0] = P + np.arange(m)
    window = int(rng.choice([0, 0, 512]))
    R = int(rng.choice([1, 4, 8]))
    for o in (host.options_reference(), host.options_mi355x(R, int(rng.choice([256, 512, 1024])))):
        tiles, jobs, parts = host.plan_tiles(np.array(trees, abi.TREE_DT), 4, window, pos if window else None, o)
        R_ = o.rows_per_tile
        # every (tree, row tile) is covered once; its ranges partition [k0, P); the last owns the batch keys
        by = {}
        for x in tiles:
            by.setdefault((int(x["tree"]), int(x["r0"])), []).append(x)
        want_keys = {(ti, base + r) for ti, (base, P, _, m) in enumerate(trees) for r in range(0, m, R_)}
        assert set(by) == want_keys
        used_parts = []
        for (ti, r0), xs in by.items():
            base, P, _, m = trees[ti]
            # records may come in any order (the balanced rule lists the owners of the batch keys first); a group's
            # partial records are numbered in range order, which is the order they merge in
            xs.sort(key=lambda x: (int(x["k0"]), int(x["last"])))
            if len(xs) > 1:
                assert [int(x["part"]) for x in xs] == list(range(int(xs[0]["part"]), int(xs[0]["part"]) + len(xs)))
            k = int(xs[0]["k0"])
            if window == 0:
                assert k == 0
            for i, x in enumerate(xs):
                assert int(x["k0"]) == k and int(x["k1"]) > k or P == k
                k = int(x["k1"])
                assert int(x["last"]) == (1 if i == len(xs) - 1 else 0)
                if len(xs) > 1:
                    used_parts.append(int(x["part"]))
                    if i:
                        # reference rule: steps from k0 (gemma.h:109); balanced rule: absolute page multiples
                        off = 0 if o.balanced else int(xs[0]["k0"])
                        assert (int(x["k0"]) - off) % o.granule == 0
                else:
                    assert int(x["part"]) == -1
            assert k == P
        assert sorted(used_parts) == list(range(parts))
        # merge jobs name consecutive parts in range order
        seen = 0
        for jb in jobs:
            assert int(jb["part0"]) == seen and int(jb["nparts"]) >= 2
            seen += int(jb["nparts"])
        assert seen == parts


def _check_tiled_partition(trees, tiles, jobs, parts, o):
    by = {}
    for x in tiles:
        by.setdefault((int(x["tree"]), int(x["r0"])), []).append(x)
    assert set(by) == {(ti, b + r) for ti, (b, P, _, m) in enumerate(trees) for r in range(0, m, 128)}
    numbered, cut = [], 0
    for (ti, r0), xs in by.items():
        base, P, _, m = trees[ti]
        k, b = 0, 0      # cached keys and batch rows handed out so far
        for i, x in enumerate(xs):
            last = int(x["last"])
            assert int(x["k0"]) == k and int(x["k1"]) >= k
            assert int(x["k0"]) % o.granule == 0
            k = int(x["k1"])
            if last:                                   # the part takes batch rows from where the one before it stopped
                assert k == P and int(x["b0"]) == b
                if last >= 2:                          # ... up to row last - 2, on a granule boundary, and a later part goes on
                    assert i < len(xs) - 1 and last - 2 >= b and (last - 1) % o.granule == 0
                    b, cut = last - 1, cut + 1
            assert (last == 1) == (i == len(xs) - 1)   # the group's last part leaves its batch range open
            assert int(x["k1"]) > int(x["k0"]) or last  # no empty part
            assert (int(x["part"]) == -1) == (len(xs) == 1)
            if len(xs) > 1:
                numbered.append(int(x["part"]))
        assert k == P and b < min(m, r0 - base + 128)  # the open part begins inside the tile's own batch rows
    assert numbered == list(range(parts))          # in record order, which is the order the kernel's grid reverses
    assert sum(int(j["nparts"]) for j in jobs) == parts and all(int(j["nparts"]) >= 2 for j in jobs)
    return cut


@pytest.mark.parametrize("seed", range(8))
def test_tiled_kernel_plans_partition_every_tile(seed):
    """The balanced rule for 128-row tiles (chosen by simulating the hand-out of workgroups to slots): whatever it
    picks - no split, one chunk for all tiles, or only the shortest tiles cut - the cached ranges of a tile partition
    [0, P), its batch ranges partition the batch rows (one open range in the last part, or cut ranges in front of it),
    parts are numbered in record order and every merge job names them."""
    rng = np.random.default_rng(900 + seed)
    n = int(rng.integers(1, 5))
    trees, base = [], 0
    for _ in range(n):
        P, m = int(rng.integers(0, 40) * 256), int(rng.integers(1, 2500))
        trees.append((base, P, 0, m))
        base += m
    groups, slots = int(rng.choice([8, 16, 40])), int(rng.choice([256, 512]))
    o = host.options_mi355x(128, slots)
    if seed % 2:   # with the batch keys open to cuts, and fixed costs low enough that some are made
        o.cut_batch, o.item_steps, o.part_steps = 1, int(rng.choice([1, 3, 6])), int(rng.choice([0, 4, 8]))
    tiles, jobs, parts = host.plan_tiles(np.array(trees, abi.TREE_DT), groups, 0, None, o)
    _check_tiled_partition(trees, tiles, jobs, parts, o)


@pytest.mark.parametrize("trees,groups,slots", [
    ([(0, 0, 0, 2048)], 16, 256),                      # one prompt's first chunk: batch rows only
    ([(0, 0, 0, 1500)], 8, 256),                       # ragged end
    ([(0, 384, 0, 2048)], 16, 256),                    # a part that ends the cached keys and begins the batch rows
    ([(0, 0, 0, 1100), (1100, 256, 0, 900)], 8, 512),  # two prompts
    ([(0, 0, 0, 4096)], 4, 256),
])
def test_cut_batch_plans_partition_the_batch_rows(trees, groups, slots):
    """With cut_batch (and fixed costs low enough that cuts are made) a tile's batch rows are cut like its cached keys:
    parts with last = their last row + 2 in front of one open part, batch ranges that follow each other without a gap."""
    o = host.options_mi355x(128, slots)
    o.cut_batch, o.item_steps, o.part_steps = 1, 2, 2
    tiles, jobs, parts = host.plan_tiles(np.array(trees, abi.TREE_DT), groups, 0, None, o)
    assert _check_tiled_partition(trees, tiles, jobs, parts, o) > 0
    o.cut_batch = 0
    tiles, _, _ = host.plan_tiles(np.array(trees, abi.TREE_DT), groups, 0, None, o)
    assert all(int(x["last"]) in (0, 1) for x in tiles)


def test_a_round_and_a_quarter_of_workgroups_is_cut_at_its_short_end():
    """A 2048-row causal chunk over 6144 cached keys, 40 workgroups per tile, 512 slots: 640 workgroups. Unsplit,
    128 of them would run after the first 512, nearly alone. The plan cuts the 4 tiles with the fewest keys (the
    first rows), the last-dispatched one into the most parts, and leaves 12 x 40 = 480 <= 512 whole workgroups."""
    trees = np.array([(0, 6144, 0, 2048)], abi.TREE_DT)
    tiles, jobs, parts = host.plan_tiles(trees, 40, 0, None, host.options_mi355x(128, 512))
    per_tile = [int((tiles["r0"] == r).sum()) for r in range(0, 2048, 128)]
    assert per_tile[4:] == [1] * 12 and all(p >= 2 for p in per_tile[:4])
    assert per_tile[:4] == sorted(per_tile[:4], reverse=True) and per_tile[0] > per_tile[3]
    assert len(jobs) == 4 and parts == sum(per_tile[:4])
    # exactly one round of workgroups (16 x 32 = 512): nothing to gain, nothing is cut
    tiles, jobs, parts = host.plan_tiles(trees, 32, 0, None, host.options_mi355x(128, 512))
    assert len(tiles) == 16 and parts == 0
    # a chunk with nothing cached has no range to cut
    tiles, jobs, parts = host.plan_tiles(np.array([(0, 0, 0, 2048)], abi.TREE_DT), 40, 0, None, host.options_mi355x(128, 512))
    assert len(tiles) == 16 and parts == 0


def test_balanced_rule_equalises_keys_per_workgroup():
    """16 sequences of 512..8192 keys: the reference rule gives every sequence the same
    number of splits; the balanced rule gives every workgroup about the same key count."""
    rng = np.random.default_rng(2)
    lens = rng.integers(512, 8193, 16)
    trees = np.array([(i, int(L), 0, 1) for i, L in enumerate(lens)], abi.TREE_DT)
    ref_t, _, _ = host.plan_tiles(trees, 4, 0, None, host.options_reference())
    bal_t, _, _ = host.plan_tiles(trees, 4, 0, None, host.options_mi355x(1, 1024))
    ref_sz = np.array([int(x["k1"] - x["k0"]) for x in ref_t])
    bal_sz = np.array([int(x["k1"] - x["k0"]) for x in bal_t])
    assert ref_sz.max() / ref_sz.min() > 4
    assert bal_sz.max() / np.median(bal_sz) < 1.3
    assert 0.5 * 1024 / 4 <= len(bal_t) <= 1.5 * 1024 / 4


# ---------------------------------------------------------------- pool: allocator and copy-on-write lists
def _conservation(e, n_blocks, slots):
    """Sum of refcounts == sum of list memberships; free + live == n_blocks."""
    member = np.zeros(n_blocks, int)
    for s in slots:
        if e.slot_len(s) >= 0:
            for b in e.slot_blocks(s):
                member[b] += 1
    refs = np.array([e.block_ref(b) for b in range(n_blocks)])
    assert (refs == member).all()
    assert e.free_blocks() + int((refs > 0).sum()) == n_blocks


def test_allocator_hands_out_block_zero_first_and_conserves():
    e = host.Engine(8, 16, 4)
    s = e.slot_alloc()
    e.pass_begin([host.make_spec(parent=-1, save=s, root_len=40)])
    e.pass_commit()
    assert list(e.slot_blocks(s)) == [0, 1, 2] and e.slot_len(s) == 40 and e.free_blocks() == 5
    _conservation(e, 8, [s])
    e.slot_reset(s)
    assert e.free_blocks() == 8 and e.slot_len(s) == 0
    # released blocks are reused last-in first-out (model.h:731-733)
    e.pass_begin([host.make_spec(save=s, root_len=16)])
    e.pass_commit()
    assert list(e.slot_blocks(s)) == [2]


def test_target_blocks_cases_match_the_restatement():
    """In place with sole ownership / shared partial block (copy on write) / block-aligned append."""
    for (P, n_new, fork, in_place) in [(40, 1, False, True), (40, 1, True, True), (40, 30, True, False), (32, 5, True, True),
                                       (32, 5, False, True), (0, 20, False, False), (47, 1, False, True), (48, 1, False, True)]:
        e = host.Engine(32, 16, 4)
        pool = ho.Pool(32, 16)
        a, b = e.slot_alloc(), e.slot_alloc()
        parent_blocks = []
        if P:
            e.pass_begin([host.make_spec(save=a, root_len=P)])
            e.pass_commit()
            parent_blocks, _ = ho.target_blocks(pool, [], 0, 0, P, False)
        assert list(e.slot_blocks(a)) == parent_blocks
        if fork:
            e.slot_fork(a, b)
            for blk in parent_blocks:
                pool.retain(blk)
        dst = a if in_place else b
        if not in_place and not fork:
            pass
        want_new = ho.target_new_blocks(pool, parent_blocks if P else None, P, P, P + n_new, in_place)
        spec = host.make_spec(parent=a if P else -1, save=dst, root_len=n_new)
        assert e.pass_blocks([spec]) == want_new
        free0 = e.free_blocks()
        ps = e.pass_begin([spec])
        want_blocks, want_cow = ho.target_blocks(pool, parent_blocks, P, P, P + n_new, in_place and P > 0)
        assert free0 - e.free_blocks() == want_new            # pass_kv_tokens == blocks actually taken
        assert [tuple(x) for x in ps["cow"].tolist()] == want_cow
        assert _as_tuples(ps["saves"]) == ho.kv_saves(0, P, n_new, want_blocks, 16)
        assert list(ps["table"]) == parent_blocks[:(P + 15) // 16]
        e.pass_commit()
        assert list(e.slot_blocks(dst)) == want_blocks and e.slot_len(dst) == P + n_new
        _conservation(e, 32, [a, b])


def test_failed_pass_leaves_slots_and_pool_untouched():
    e = host.Engine(6, 16, 4)
    a, b = e.slot_alloc(), e.slot_alloc()
    e.pass_begin([host.make_spec(save=a, root_len=50)])
    e.pass_commit()
    before = (list(e.slot_blocks(a)), e.slot_len(a), e.free_blocks())
    with pytest.raises(abi.EspError, match="KV cache full"):
        e.pass_begin([host.make_spec(parent=a, save=b, root_len=64)])
    with pytest.raises(abi.EspError, match="two trees save into one slot"):
        e.pass_begin([host.make_spec(parent=a, save=b, root_len=1), host.make_spec(parent=a, save=b, root_len=1)])
    with pytest.raises(abi.EspError, match="work slot must differ"):
        e.pass_begin([host.make_spec(parent=a, save=a, work=a, root_len=1)])
    with pytest.raises(abi.EspError, match="invalid parent slot"):
        e.pass_begin([host.make_spec(parent=3, root_len=1)])
    with pytest.raises(abi.EspError, match="empty tree"):
        e.pass_begin([host.make_spec(parent=a)])
    assert (list(e.slot_blocks(a)), e.slot_len(a), e.free_blocks()) == before
    # an aborted pass (the device work failed) gives its blocks back
    e.pass_begin([host.make_spec(parent=a, save=b, root_len=20)])
    assert e.free_blocks() < before[2]
    e.pass_abort()
    assert (list(e.slot_blocks(a)), e.slot_len(a), e.free_blocks()) == before and e.slot_len(b) == 0
    _conservation(e, 6, [a, b])


def test_fork_shares_blocks_and_copy_on_write_diverges():
    e = host.Engine(16, 16, 4)
    a, b = e.slot_alloc(), e.slot_alloc()
    e.pass_begin([host.make_spec(save=a, root_len=40)])
    e.pass_commit()
    e.slot_fork(a, b)
    assert list(e.slot_blocks(a)) == list(e.slot_blocks(b))
    assert all(e.block_ref(x) == 2 for x in e.slot_blocks(a))
    ps = e.pass_begin([host.make_spec(parent=a, save=a, root_len=1), host.make_spec(parent=b, save=b, root_len=1)])
    # both partial blocks are shared: each append copies block 2 into a fresh one
    assert len(ps["cow"]) == 2 and all(src == 2 for src, _ in ps["cow"].tolist())
    e.pass_commit()
    la, lb = list(e.slot_blocks(a)), list(e.slot_blocks(b))
    assert la[:2] == lb[:2] and la[2] != lb[2] and e.block_ref(2) == 0
    _conservation(e, 16, [a, b])


@pytest.mark.parametrize("seed", range(6))
def test_random_slot_histories_keep_every_slot_readable(seed):
    """Model-based: random appends (in place, into another slot, after forks), aborted and refused passes, resets.
    A toy pool holds one token id per (block, position); the pass's own records drive it - copy-on-write pairs
    first, then the saves - and after every step each slot must read back, through its block list, exactly the
    tokens it logically holds, the parent's table must read the parent's tokens, and the blocks must add up."""
    rng = np.random.default_rng(300 + seed)
    bt = int(rng.choice([16, 32]))
    n_blocks, n_slots = int(rng.integers(10, 40)), 5
    e = host.Engine(n_blocks, bt, n_slots)
    slots = [e.slot_alloc() for _ in range(n_slots)]
    truth = {s: [] for s in slots}
    pool = np.full((n_blocks, bt), -1, np.int64)
    next_tok = [1]
    # sliding layers: a second toy pool of one ring per slot (forest.h:2657-2700); what a slot's next row can see
    # there - its last W - 1 positions - must read back too
    W = int(rng.integers(5, 120))
    rb = (W + bt - 1) // bt + int(rng.integers(0, 2))
    ring = np.full((n_slots * rb, bt), -1, np.int64)

    def read(blocks, n):
        return [int(x) for x in pool[list(blocks)].reshape(-1)[:n]] if n else []

    def check_all():
        for s in slots:
            assert e.slot_len(s) == len(truth[s])
            assert read(e.slot_blocks(s), len(truth[s])) == truth[s], (seed, s)
            L = len(truth[s])
            for p_ in range(max(0, L - W + 1), L):
                assert ring[s * rb + (p_ // bt) % rb, p_ % bt] == truth[s][p_], (seed, s, p_)
        _conservation(e, n_blocks, slots)

    for step in range(120):
        op = rng.choice(["pass", "pass", "pass", "fork", "reset"])
        if op == "fork":
            a, b = (int(x) for x in rng.choice(slots, 2, replace=False))
            e.slot_reset(b)
            e.slot_fork(a, b)
            truth[b] = list(truth[a])
            ring[b * rb:(b + 1) * rb] = ring[a * rb:(a + 1) * rb]   # a fork copies the whole ring (forest.h:127-137)
        elif op == "reset":
            a = int(rng.choice(slots))
            e.slot_reset(a)
            truth[a] = []
        else:
            # up to 3 trees, distinct destinations; a tree extends a parent in place, or into an empty slot, or starts fresh
            dsts = [int(x) for x in rng.choice(slots, int(rng.integers(1, 4)), replace=False)]
            specs, plan = [], []
            for d in dsts:
                n_new = int(rng.integers(1, 50))
                kind = rng.choice(["inplace", "from", "fresh"])
                if kind == "inplace" and truth[d]:
                    parent = d
                elif kind == "from":
                    parent = int(rng.choice(slots))
                    if not truth[parent] or parent == d or parent in dsts:   # a parent that another tree rewrites is left out
                        parent = -1
                else:
                    parent = -1
                if parent != d:
                    e.slot_reset(d)
                    truth[d] = []
                specs.append(host.make_spec(parent=parent, save=d, root_len=n_new))
                plan.append((parent, d, n_new))
            before = (pool.copy(), {s: list(e.slot_blocks(s)) for s in slots}, e.free_blocks())
            try:
                ps = e.pass_begin(specs)
            except abi.EspError:
                assert ({s: list(e.slot_blocks(s)) for s in slots}, e.free_blocks()) == before[1:]   # refused: nothing moved
                check_all()
                continue
            rows = {}
            for t, (parent, d, n_new) in zip(ps["trees"], plan):
                assert int(t["M"]) == n_new and int(t["P"]) == (len(truth[parent]) if parent >= 0 else 0)
                toks = list(range(next_tok[0], next_tok[0] + n_new))
                next_tok[0] += n_new
                for r, tok in enumerate(toks):
                    rows[int(t["base"]) + r] = tok
                plan[plan.index((parent, d, n_new))] = (parent, d, toks)
                if parent >= 0:   # what the attention of this tree reads through its table: the parent's tokens
                    nb = (len(truth[parent]) + bt - 1) // bt
                    tab = ps["table"][int(t["table"]):int(t["table"]) + nb]
                    cowmap = {int(dst): int(src) for src, dst in ps["cow"].tolist()}
                    assert [int(x) for x in pool[[cowmap.get(int(b), int(b)) for b in tab]].reshape(-1)[:len(truth[parent])]] == truth[parent]
            rg = e.pass_rings(W, rb)
            want = ho.ring_plan([(int(t["base"]), int(t["P"]), int(t["M"]), parent, [(d, len(toks))])
                                 for t, (parent, d, toks) in zip(ps["trees"], plan)], W, rb, bt)
            assert [tuple(int(x) for x in t) for t in rg["trees"]] == want[0]
            assert [tuple(int(x) for x in t) for t in rg["saves"]] == want[1]
            assert [tuple(c) for c in rg["copies"].tolist()] == want[2]
            ring_before = ring.copy()
            for src, dst in rg["copies"].tolist():                   # copies, then saves
                ring[dst] = ring[src]
            for sv in rg["saves"]:
                ring[int(sv["block"]), int(sv["pos"])] = rows[int(sv["src_row"])]
            for src, dst in ps["cow"].tolist():
                pool[dst] = pool[src]
            for sv in ps["saves"]:
                pool[int(sv["block"]), int(sv["pos"])] = rows[int(sv["src_row"])]
            if rng.integers(0, 4) == 0:
                e.pass_abort()
                pool[:] = before[0]
                ring[:] = ring_before      # an in-place chunk's saves reuse ring cells the slot still needs if it does not advance
                assert ({s: list(e.slot_blocks(s)) for s in slots}, e.free_blocks()) == before[1:]
            else:
                e.pass_commit()
                new_truth = {d: (list(truth[parent]) if parent >= 0 else []) + toks for parent, d, toks in plan}
                truth.update(new_truth)
        check_all()


# ---------------------------------------------------------------- rows of verify trees
def test_leaf_hosting_and_descriptors_match_the_restatement():
    rng = np.random.default_rng(5)
    for _ in range(30):
        NL = int(rng.integers(1, 6))
        leaves = []
        for _ in range(NL):
            n = int(rng.integers(1, 5))
            leaves.append([int(x) for x in rng.integers(0, 3, n)])
        Tr = int(rng.integers(0, 4))
        e = host.Engine(64, 16, 2)
        s = e.slot_alloc()
        e.pass_begin([host.make_spec(save=s, root_len=33)])
        e.pass_commit()
        toks = [t for lf in leaves for t in lf]
        offs = [0]
        for lf in leaves:
            offs.append(offs[-1] + len(lf))
        ps = e.pass_begin([host.make_spec(parent=s, root_len=Tr, leaves=leaves)])
        desc, pos, M = ho.tree_rows(0, Tr, 33, toks, offs)
        assert ps["M"] == M
        assert ps["desc"].tolist() == [list(d) for d in desc]
        assert ps["pos"].tolist() == [list(p) for p in pos]
        e.pass_abort()


def test_verify_chain_is_one_tree_of_root_plus_k_rows():
    """MTP verify: leaf i = first i + 1 drafts; prefixes are hosted by the longest leaf, so the
    tree has root + k rows, not k (k + 1) / 2 (forest.h:2201-2220)."""
    e = host.Engine(64, 16, 2)
    s = e.slot_alloc()
    e.pass_begin([host.make_spec(save=s, root_len=100)])
    e.pass_commit()
    drafts = [5, 6, 7]
    leaves = [drafts[:i + 1] for i in range(3)]
    ps = e.pass_begin([host.make_spec(parent=s, save=s, root_len=1, leaves=leaves, commit_chain=3)])
    assert ps["M"] == 4
    assert ps["desc"].tolist() == [[0, 0, 0, 0], [1, 0, 1, 0], [1, 0, 1, 0], [1, 0, 1, 0]]
    assert ps["pos"][:, 0].tolist() == [100, 101, 102, 103]
    # root row and the chain rows are all saved at the positions they take if committed
    assert [(int(x["src_row"]), int(x["pos"])) for x in ps["saves"]] == [(0, 4), (1, 5), (2, 6), (3, 7)]
    e.pass_commit()
    assert e.slot_len(s) == 101


def test_row_table_matches_the_restatement_and_refuses_a_third_slot():
    """kv_row_table (src/model/impl/forest.h:1737-1749) through the C shim against its restatement."""
    rng = np.random.default_rng(5)
    rows = 23
    saves = [(int(r), int(rng.integers(0, 50)), int(rng.integers(0, 16)), 0) for r in rng.permutation(rows)[:17]]
    saves += [(saves[3][0], 7, 9, 0), (saves[8][0], 8, 1, 0)]          # two rows go to a second slot
    got = host.row_table(np.array(saves, abi.KVSAVE_DT), rows)
    assert got.tolist() == ho.kv_row_table(saves, rows)
    assert (got[[r for r in range(rows) if r not in {s[0] for s in saves}]] == -1).all()
    with pytest.raises(abi.EspError):
        host.row_table(np.array(saves + [(saves[3][0], 1, 1, 0)], abi.KVSAVE_DT), rows)
    with pytest.raises(ValueError):
        ho.kv_row_table(saves + [(saves[3][0], 1, 1, 0)], rows)
    assert host.row_table(np.zeros(0, abi.KVSAVE_DT), 4).tolist() == [[-1] * 4] * 4


def test_open_ended_marks_exactly_the_ranges_that_end_at_the_cached_length():
    trees = np.array([(0, 5000, 0, 1), (1, 40, 400, 1), (2, 0, 500, 1)], abi.TREE_DT)
    tiles, jobs, n_parts = host.plan_tiles(trees, 4, 0, None, host.options_mi355x(1, 64))
    opened = host.open_ended(tiles, trees)
    last = tiles["k1"] == trees["P"][tiles["tree"]]
    assert last.sum() == 3 and (tiles["last"][last] == 1).all()        # one per tree, and it is the part with the batch keys
    assert (opened["k1"][last] == 2**31 - 1).all() and (opened["k1"][~last] == tiles["k1"][~last]).all()
    for f in ("tree", "r0", "k0", "part", "last", "b0", "pad"):
        assert (opened[f] == tiles[f]).all()


def test_slot_file_round_trip_layout_and_refusals(tmp_path):
    """The reference's checkpoint format, KV section (src/model/model.mm:600-752): 120-byte header with magic
    0x554b5043 and version 4, then the blocks layer-major; a file of the wrong size, version or with
    sections of other subsystems is refused (slot_load's -1, :700-714)."""
    import struct
    rng = np.random.default_rng(6)
    n_layers, n_blocks, bt, kvw = 3, 5, 16, 2 * 128
    kv = rng.integers(0, 65536, (n_layers, n_blocks, 2 * bt * kvw), dtype=np.uint16)
    path = tmp_path / "slot.ckpt"
    host.slot_file_save(path, 70, 70, n_layers, kv)
    raw = path.read_bytes()
    assert len(raw) == 120 + kv.nbytes
    magic, version, length, next_pos = struct.unpack_from("<IIii", raw, 0)
    assert (magic, version, length, next_pos) == (0x554B5043, 4, 70, 70)
    assert struct.unpack_from("<iii", raw, 36) == (n_blocks, n_layers, 0)          # n_blocks, n_layers, n_linear
    assert struct.unpack_from("<Q", raw, 48)[0] == 2 * bt * kvw * 2                # block_bytes
    assert raw[120:] == kv.tobytes()                                               # layer-major, logical order
    got = host.slot_file_load(path, bt)
    assert (got["len"], got["next_pos"], got["n_blocks"], got["n_layers"]) == (70, 70, n_blocks, n_layers)
    assert np.array_equal(got["kv"].view(np.uint16).reshape(kv.shape), kv)
    # refusals
    assert host.slot_file_load(tmp_path / "missing.ckpt", bt) is None
    (tmp_path / "short.ckpt").write_bytes(raw[:-2])
    assert host.slot_file_load(tmp_path / "short.ckpt", bt) is None
    bad = bytearray(raw)
    struct.pack_into("<I", bad, 4, 3)                                              # another version
    (tmp_path / "v3.ckpt").write_bytes(bytes(bad))
    assert host.slot_file_load(tmp_path / "v3.ckpt", bt) is None
    bad = bytearray(raw)
    struct.pack_into("<i", bad, 44, 2)                                             # n_linear: state of other layers follows
    (tmp_path / "lin.ckpt").write_bytes(bytes(bad))
    assert host.slot_file_load(tmp_path / "lin.ckpt", bt) is None
    bad = bytearray(raw)
    struct.pack_into("<i", bad, 8, n_blocks * bt + 1)                              # more tokens than the blocks hold
    (tmp_path / "len.ckpt").write_bytes(bytes(bad))
    assert host.slot_file_load(tmp_path / "len.ckpt", bt) is None
    # an empty slot is a header alone
    host.slot_file_save(tmp_path / "empty.ckpt", 0, 0, n_layers, np.zeros((n_layers, 0, 2 * bt * kvw), np.uint16))
    e = host.slot_file_load(tmp_path / "empty.ckpt", bt)
    assert e["n_blocks"] == 0 and (tmp_path / "empty.ckpt").stat().st_size == 120


def test_slot_file_ring_section(tmp_path):
    """The file's last section (src/model/model.mm:664-669, 737-742): after the KV blocks, per sliding layer the
    slot's ring, r_blocks blocks of rblock_bytes; counts in the header's last three fields (:611-612)."""
    import struct
    rng = np.random.default_rng(7)
    n_layers, n_blocks, bt, kvw_g, kvw_s, r_layers, rb = 2, 4, 16, 2 * 512, 8 * 256, 5, 3
    kv = rng.integers(0, 65536, (n_layers, n_blocks, 2 * bt * kvw_g), dtype=np.uint16)
    rings = rng.integers(0, 65536, (r_layers, rb, 2 * bt * kvw_s), dtype=np.uint16)
    path = tmp_path / "g4.ckpt"
    host.slot_file_save_rings(path, 60, 61, n_layers, kv, rings)
    raw = path.read_bytes()
    assert len(raw) == 120 + kv.nbytes + rings.nbytes
    assert struct.unpack_from("<iiQ", raw, 104) == (r_layers, rb, 2 * bt * kvw_s * 2)
    assert raw[120:120 + kv.nbytes] == kv.tobytes() and raw[120 + kv.nbytes:] == rings.tobytes()
    got = host.slot_file_load_rings(path, bt)
    assert (got["len"], got["next_pos"], got["r_layers"], got["r_blocks"]) == (60, 61, r_layers, rb)
    assert np.array_equal(got["kv"].view(np.uint16).reshape(kv.shape), kv)
    assert np.array_equal(got["rings"].view(np.uint16).reshape(rings.shape), rings)
    assert host.slot_file_load(path, bt) is None                  # a loader without ring pools refuses it
    (tmp_path / "short.ckpt").write_bytes(raw[:-2])
    assert host.slot_file_load_rings(tmp_path / "short.ckpt", bt) is None
    bad = bytearray(raw)
    struct.pack_into("<i", bad, 104, 0)                           # ring blocks without ring layers
    (tmp_path / "norl.ckpt").write_bytes(bytes(bad))
    assert host.slot_file_load_rings(tmp_path / "norl.ckpt", bt) is None
    # a file without rings loads through either call
    host.slot_file_save(tmp_path / "plain.ckpt", 60, 61, n_layers, kv)
    p = host.slot_file_load_rings(tmp_path / "plain.ckpt", bt)
    assert p["r_layers"] == 0 and p["rings"].size == 0 and np.array_equal(p["kv"].view(np.uint16).reshape(kv.shape), kv)


def test_verify_commit_takes_the_kept_chain_rows_into_the_slot():
    """run_commit's block-pool side (src/model/impl/forest.h:4846-4861, 5058-5069): after a verify pass that kept a
    chain of k draft rows, the first n of them join the slot - they already sit at positions len .. len + n - 1 -
    and only while no other pass has begun; a fork does not inherit them (model.mm:551)."""
    bt = 16
    e = host.Engine(16, bt, 3)
    a, b, c = (e.slot_alloc() for _ in range(3))
    pool = np.full((16, bt), -1, np.int64)

    def run(specs, tokens):
        ps = e.pass_begin(specs)
        for src, dst in ps["cow"].tolist():
            pool[dst] = pool[src]
        for sv in ps["saves"]:
            pool[int(sv["block"]), int(sv["pos"])] = tokens[int(sv["src_row"])]
        e.pass_commit()
        return ps

    def read(s, n):
        return [int(x) for x in pool[list(e.slot_blocks(s))].reshape(-1)[:n]]

    run([host.make_spec(save=a, root_len=30)], list(range(100, 130)))
    assert e.slot_chain(a) == 0
    drafts = [7, 8, 9]
    ps = run([host.make_spec(parent=a, save=a, root_len=1, leaves=[drafts[:i + 1] for i in range(3)], commit_chain=3)],
             [200, 201, 202, 203])                                      # row 0 the pending token, rows 1..3 the chain
    assert ps["M"] == 4 and e.slot_len(a) == 31 and e.slot_next_pos(a) == 31 and e.slot_chain(a) == 3
    assert [(int(s_["src_row"]), int(s_["pos"])) for s_ in ps["saves"]] == [(0, 30 % bt), (1, 31 % bt), (2, 0), (3, 1)]
    with pytest.raises(abi.EspError):
        e.chain_commit(a, 4)                                            # more than the pass kept
    assert e.slot_chain(a) == 3                                         # a refused request changes nothing
    e.slot_fork(a, b)
    assert e.slot_len(b) == 31 and e.slot_chain(b) == 0 and len(e.slot_blocks(b)) == 2   # the fork: [0, len) only
    with pytest.raises(abi.EspError):
        e.chain_commit(b, 1)
    e.chain_commit(a, 2)
    assert e.slot_len(a) == 33 and e.slot_next_pos(a) == 33 and e.slot_chain(a) == 0
    assert read(a, 33) == list(range(100, 130)) + [200, 201, 202]
    with pytest.raises(abi.EspError):
        e.chain_commit(a, 1)                                            # the rest of the chain was dropped
    # the next token goes where the third draft row sat; the fork still reads its own 31
    run([host.make_spec(parent=a, save=a, root_len=1)], [300])
    assert read(a, 34) == list(range(100, 130)) + [200, 201, 202, 300] and read(b, 31) == list(range(100, 130)) + [200]
    # chain rows are only committable until another pass begins, whichever slots it names
    run([host.make_spec(parent=a, save=a, root_len=1, leaves=[[5]], commit_chain=1)], [301, 302])
    assert e.slot_chain(a) == 1
    run([host.make_spec(save=c, root_len=3)], [400, 401, 402])
    assert e.slot_chain(a) == 0
    with pytest.raises(abi.EspError):
        e.chain_commit(a, 1)
    e.chain_commit(a, 0)                                                # declining is always allowed
    assert e.slot_len(a) == 35
    _conservation(e, 16, [a, b, c])


def test_slots_of_the_pending_pass_cannot_be_freed_reset_or_forked_over():
    """Between pass_begin and commit / abort the pass's parent, save and work slots stay as they are: a commit would
    otherwise write the pass's block lists into a slot the caller has given back."""
    e = host.Engine(32, 16, 4)
    a, b, c, d = (e.slot_alloc() for _ in range(4))
    e.pass_begin([host.make_spec(save=a, root_len=20)])
    e.pass_commit()
    e.pass_begin([host.make_spec(parent=a, save=b, work=c, root_len=5)])
    free = e.free_blocks()
    for s in (a, b, c):
        assert e.slot_free(s) != 0 and e.slot_reset(s) != 0, s
    assert e.slot_fork(d, b) != 0          # b would be overwritten under the pass
    assert e.slot_fork(a, d) == 0          # reading the parent into a slot outside the pass is fine
    assert e.slot_reset(d) == 0
    assert e.free_blocks() == free and e.slot_len(a) == 20
    e.pass_commit()
    assert e.slot_len(b) == 25 and e.slot_len(c) == 25
    assert e.slot_free(b) == 0 and e.slot_free(c) == 0 and e.slot_free(a) == 0
    assert e.free_blocks() == 32


def test_slot_adopt_gives_a_loaded_checkpoint_its_slot_and_blocks():
    """slot_load's engine side (src/model/model.mm:694-752): counts that do not fit -> -1, no room -> -2, else a slot
    whose fresh blocks the caller fills; the slot then behaves like any other (decode appends in place)."""
    e = host.Engine(10, 16, 2, max_ctx=1000)
    assert e.slot_adopt(33, 33, 2) == -1           # 33 positions need 3 blocks
    assert e.slot_adopt(2000, 2000, 200) == -1     # beyond max_ctx
    assert e.slot_adopt(100, 100, 11) == -2        # the pool has 10 blocks
    s = e.slot_adopt(33, 40, 3)
    assert s >= 0 and e.slot_len(s) == 33 and e.slot_next_pos(s) == 40 and e.free_blocks() == 7
    blocks = e.slot_blocks(s)
    assert len(set(blocks.tolist())) == 3 and all(e.block_ref(int(b)) == 1 for b in blocks)
    ps = e.pass_begin([host.make_spec(parent=s, save=s, root_len=1)])
    assert ps["pos"][0, 0] == 40 and len(ps["cow"]) == 0 and ps["saves"][0]["block"] == blocks[2] and ps["saves"][0]["pos"] == 1
    e.pass_commit()
    t = e.slot_adopt(16, 16, 1)
    assert t >= 0 and e.slot_adopt(1, 1, 1) == -2  # no slot left
    e.slot_free(s)
    e.slot_free(t)
    assert e.free_blocks() == 10


def test_noncausal_root_rows_are_described_as_seeing_the_whole_root():
    """A noncausal root (the reference's pplx heads, src/model/impl/forest.h:2402-2403): every root row's descriptor
    names the whole root as ancestors (anc_len = root_len), so row i also sees rows after it
    (kernels/40_attention.metal:104-113). Such a tree is a root alone."""
    e = host.Engine(8, 16, 2)
    ps = e.pass_begin([host.make_spec(root_len=5, noncausal=1)])
    assert ps["M"] == 5 and (ps["desc"][:, 2] == 5).all() and (ps["desc"][:, 0] == 0).all()
    assert ps["pos"][:, 0].tolist() == [0, 1, 2, 3, 4]
    e.pass_abort()
    s = e.slot_alloc()
    for bad in (dict(save=s), dict(parent=s), dict(leaves=[[1]])):
        with pytest.raises(abi.EspError, match="noncausal"):
            e.pass_begin([host.make_spec(root_len=5, noncausal=1, **bad)])
