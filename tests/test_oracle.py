"""Pins the CPU checker (oracle/) before anything is compared against it.

The reference holds no golden vectors and no CPU implementation for this path
(its attention is Metal only), so the checker is pinned by what the
mathematics fixes: a float64 brute force over gathered keys with an explicit
mask matrix, torch's CPU scaled_dot_product_attention, closed forms, and
invariants (split count, page permutation, window >= context, chunking).
Each check is chosen so that a plausible mistake fails it: a wrong mask
comparison, a transposed page index, a dropped rescale, l summed from rounded
P, K/V planes swapped.
"""
import numpy as np
import pytest
import torch

from espetero_amd import abi, host, synth
from oracle import binding as ob
from oracle import host_oracle as ho

from helpers import TOL, brute, f32, max_abs, oracle_direct, small_case, tol_for


# ---------------------------------------------------------------- conversions
def test_half_to_float_all_values():
    L = ob.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.esp_oracle_h2f(int(b)) for b in bits], np.float32)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all()


def test_float_to_half_rne_matches_numpy():
    L = ob.lib()
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(4000).astype(np.float32),
        (rng.standard_normal(2000) * 1e-5).astype(np.float32),   # subnormal halves
        (rng.standard_normal(500) * 7e4).astype(np.float32),     # overflow
        np.array([0.0, -0.0, 65504.0, 65520.0, 65519.99, 5.9604645e-08, 2.9802322e-08, 2.98023224e-08 * 1.0000001,
                  1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11, np.inf, -np.inf], np.float32)])
    want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.esp_oracle_f2h(float(x)) for x in xs], np.uint16)
    assert (got == want).all()


def test_bf16_roundtrip_and_rne():
    L = ob.lib()
    rng = np.random.default_rng(1)
    xs = rng.standard_normal(3000).astype(np.float32)
    want = torch.from_numpy(xs).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.esp_oracle_f2bf(float(x)) for x in xs], np.uint16)
    assert (got == want).all()
    assert (ob.from_f32(xs, abi.ESP_BF16) == want).all()
    back = np.array([L.esp_oracle_bf2f(int(b)) for b in got], np.float32)
    assert (back == ob.to_f32(got, abi.ESP_BF16)).all()


# ---------------------------------------------------------------- brute force / library cross-checks
CASES = [
    dict(seqs=((70, 1), (33, 1))),                                   # decode, ragged page tails
    dict(seqs=((0, 5),)),                                            # first prefill chunk: no cache at all
    dict(seqs=((37, 19), (16, 3))),                                  # chunked prefill against a cache
    dict(seqs=((50, 4),), desc_fn=lambda M: synth.verify_desc(M, 1)),  # verify: root 1 + chain 3
    dict(seqs=((90, 6), (10, 1)), window=32),                        # sliding window, block lists
    dict(seqs=((90, 1), (200, 1)), window=64, ring_layer=True),      # sliding window, slot rings
    dict(seqs=((41, 7),), H=10, Hkv=2, dtype=abi.ESP_BF16),          # GQA 5, bf16
    dict(seqs=((33, 2),), H=4, Hkv=2, HD=256),                       # head_dim 256
    dict(seqs=((40, 3),), H=8, Hkv=1, HD=512),                       # head_dim 512, GQA 8 (Gemma 4 global layers)
    dict(seqs=((64, 9),), bt=64),                                    # the reference's default block size
    dict(seqs=((20, 8),), H=4, Hkv=2, bidi=1, desc_fn=lambda M: synth.image_desc(M, 2, 6)),  # bidirectional span
]


@pytest.mark.parametrize("kw", CASES)
def test_direct_matches_float64_brute_force(kw):
    c = small_case(seed=11, **kw)
    got = oracle_direct(c)
    assert max_abs(got, brute(c), c.params.dtype) <= tol_for(c.params.dtype, unrounded=True)


def test_direct_matches_torch_sdpa():
    """The masked case reduces to a library routine: SDPA with a boolean mask and GQA."""
    c = small_case(seed=5, seqs=((45, 6),), desc_fn=lambda M: synth.verify_desc(M, 2))
    p, t = c.params, c.trees[0]
    K, V = ob.gather_tree_kv(p, t, c.pool_ref, c.blocks, c.Kb, c.Vb)
    vis = ob.visible_mask(p, t, c.desc, c.pos)
    q = torch.from_numpy(f32(c.Q, p.dtype).reshape(c.n_rows, p.H, p.head_dim)).permute(1, 0, 2)[None]
    k = torch.from_numpy(K.astype(np.float32)).permute(1, 0, 2)[None]
    v = torch.from_numpy(V.astype(np.float32)).permute(1, 0, 2)[None]
    o = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=torch.from_numpy(vis)[None, None],
                                                         scale=float(p.scale), enable_gqa=True)
    want = o[0].permute(1, 0, 2).reshape(c.n_rows, -1).numpy()
    assert max_abs(oracle_direct(c), want, p.dtype) <= TOL


# ---------------------------------------------------------------- the tree mask, as a truth table
def test_tree_mask_truth_table():
    """Root of 3 rows + leaves {2, 1} (kernels/40_attention.metal:104-113): a row sees the cached
    keys, the whole root, and its own segment up to itself; siblings never see each other.
    q = 0 makes O the plain mean of the visible V rows, so V rows that are distinct powers of two
    per key expose the mask exactly."""
    desc, pos, M = ho.tree_rows(0, 3, 2, [7, 8, 9], [0, 2, 3])
    assert M == 6
    want = np.array([  # cols: cached 0, 1 | batch 0..5
        [1, 1, 1, 0, 0, 0, 0, 0],
        [1, 1, 1, 1, 0, 0, 0, 0],
        [1, 1, 1, 1, 1, 0, 0, 0],
        [1, 1, 1, 1, 1, 1, 0, 0],   # leaf A row 0
        [1, 1, 1, 1, 1, 1, 1, 0],   # leaf A row 1
        [1, 1, 1, 1, 1, 0, 0, 1],   # leaf B row 0: not A's rows
    ], bool)
    c = small_case(seed=3, H=2, Hkv=1, seqs=((2, 6),))
    c.desc[:] = np.asarray(desc, np.int32)
    assert (ob.visible_mask(c.params, c.trees[0], c.desc, c.pos) == want).all()
    c.Q[:] = 0
    vals = 2.0 ** np.arange(8, dtype=np.float32)          # key i -> V row filled with 2^i
    blk = c.params.bt * c.params.kv_ld
    b = int(c.blocks[0])
    for j in range(2):
        c.pool_ref[(2 * b + 1) * blk + j * c.params.kv_ld:(2 * b + 1) * blk + (j + 1) * c.params.kv_ld] = \
            ob.from_f32(np.full(c.params.kv_ld, vals[j], np.float32), abi.ESP_F16)
    for j in range(6):
        c.Vb[j] = ob.from_f32(np.full(c.params.kv_ld, vals[2 + j], np.float32), abi.ESP_F16)
    got = f32(oracle_direct(c), abi.ESP_F16)[:, 0]
    for r in range(6):
        # P = 1/n is rounded to fp16 before P.V and the output again: both < 2^-10 relative.
        assert got[r] == pytest.approx(vals[want[r]].mean(), rel=2e-3)


def test_bidirectional_span_truth_table():
    """Rows 2..5 form a span with img_end = 6 on a layer with bidi set: inside the span every row sees
    the whole span, outside it the rule stays causal (kernels/80_gemma.metal:284); without bidi the
    same descriptors are plain causal."""
    c = small_case(seed=4, H=2, Hkv=1, seqs=((1, 8),), bidi=1, desc_fn=lambda M: synth.image_desc(M, 2, 6))
    want = np.zeros((8, 9), bool)
    want[:, 0] = True                                   # the cached key
    for r in range(8):
        want[r, 1:r + 2] = True                         # causal over the batch keys
    want[2:6, 1 + 2:1 + 6] = True                       # the span sees itself whole
    assert (ob.visible_mask(c.params, c.trees[0], c.desc, c.pos) == want).all()
    c.params.bidi = 0
    causal = np.tril(np.ones((8, 8), bool))
    assert (ob.visible_mask(c.params, c.trees[0], c.desc, c.pos)[:, 1:] == causal).all()


# ---------------------------------------------------------------- closed forms
def test_closed_forms():
    c = small_case(seed=7, seqs=((40, 3),))
    p = c.params
    one = ob.from_f32(np.ones(1, np.float32), p.dtype)[0]
    # V == 1  =>  O == 1 (softmax weights sum to one)
    c1 = small_case(seed=7, seqs=((40, 3),))
    blk = p.bt * p.kv_ld
    for b in c1.blocks:
        c1.pool_ref[(2 * int(b) + 1) * blk:(2 * int(b) + 2) * blk] = one
    c1.Vb[:] = one
    o = f32(oracle_direct(c1), p.dtype)
    assert np.abs(o - 1.0).max() <= 2e-3
    # q == 0  =>  O == mean of the visible V rows
    c2 = small_case(seed=7, seqs=((40, 3),))
    c2.Q[:] = 0
    want = brute(c2)
    K, V = ob.gather_tree_kv(p, c2.trees[0], c2.pool_ref, c2.blocks, c2.Kb, c2.Vb)
    for rr in range(3):
        mean = V[:40 + rr + 1].mean(axis=0)   # [Hkv][HD]
        assert np.abs(want[rr].reshape(p.H, -1)[0] - mean[0]).max() < 1e-12
    assert max_abs(oracle_direct(c2), want, p.dtype) <= TOL
    # a single visible key  =>  O is that V row exactly (P = 1, fp16 round trip is exact)
    c3 = small_case(seed=8, seqs=((0, 1),))
    o3 = oracle_direct(c3)
    G = p.H // p.Hkv
    for h in range(p.H):
        kvh = h // G
        assert (o3[0, h * 128:(h + 1) * 128] == c3.Vb[0, kvh * 128:(kvh + 1) * 128]).all()
    # all keys equal  =>  O == mean of V (uniform weights)
    c4 = small_case(seed=9, seqs=((32, 1),))
    K0 = c4.Kb[0].copy()
    for b in c4.blocks:
        c4.pool_ref[(2 * int(b)) * blk:(2 * int(b) + 1) * blk] = np.tile(K0, p.bt)
    K, V = ob.gather_tree_kv(p, c4.trees[0], c4.pool_ref, c4.blocks, c4.Kb, c4.Vb)
    o4 = f32(oracle_direct(c4), p.dtype).reshape(p.H, -1)
    assert np.abs(o4[0] - V.mean(axis=0)[0]).max() <= TOL


def test_row_with_no_visible_key_is_zero():
    """l == 0 -> output 0 (kernels/40_attention.metal:334). A leaf row whose segment starts after
    itself and with no root and no cache sees nothing."""
    c = small_case(seed=2, seqs=((0, 2),))
    c.desc[1] = (2, 0, 0, 0)   # seg_start beyond the row: nothing visible
    o = oracle_direct(c)
    assert (o[1] == 0).all()
    assert (o[0] != 0).any()


def test_gate_is_sigmoid():
    c = small_case(seed=4, seqs=((20, 2),))
    p = c.params
    plain = f32(oracle_direct(c), p.dtype)
    gate = np.random.default_rng(0).standard_normal((c.n_rows, p.H, 2 * p.head_dim)).astype(np.float32)
    p.gate = gate.ctypes.data
    p.gate_ld, p.gate_hs, p.gate_off = p.H * 2 * p.head_dim, 2 * p.head_dim, p.head_dim
    gated = f32(oracle_direct(c), p.dtype)
    g = gate[:, :, p.head_dim:].reshape(c.n_rows, -1).astype(np.float64)
    want = brute(c) / (1.0 + np.exp(-g))
    assert np.abs(gated - want).max() <= TOL
    assert np.abs(gated - plain).max() > 1e-2
    p.gate = None


# ---------------------------------------------------------------- invariants
def _plan(c, opts_split, groups=256):
    trees = [tuple(int(x) for x in t) for t in c.trees]
    tiles, comb, parts = ho.plan_tiles(trees, c.params.Hkv, opts_split, groups=groups)
    return (np.array(tiles, abi.TILE_DT), np.array(comb, abi.COMBINE_DT) if comb else np.zeros(0, abi.COMBINE_DT), parts)


@pytest.mark.parametrize("split,groups", [(0, 256), (512, 256), (64, 4096), (32, 100000)])
def test_tiles_and_combine_match_direct(split, groups):
    """Any split of [0, P) with the merge of partial records equals the unsplit call."""
    c = small_case(seed=21, seqs=((300, 1), (129, 11)), rows_per_tile=8)
    tiles, jobs, parts = _plan(c, split, groups)
    if split == 0:
        assert parts == 0
    else:
        assert parts > 0
    got = ob.attn_tiles(c.params, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, tiles, c.trees, jobs, parts)
    assert max_abs(got, oracle_direct(c), c.params.dtype) <= 1e-3


@pytest.mark.parametrize("kw", [
    dict(seqs=((0, 300),)),                                                            # batch keys only
    dict(seqs=((70, 200), (0, 150))),                                                  # a part that ends the cached keys and begins the batch keys
    dict(seqs=((0, 260),), window=60),                                                 # cuts around the window's lower edge
    dict(seqs=((20, 220),), bidi=1, desc_fn=lambda M: synth.image_desc(M, 90, 170)),   # rows that see beyond their own tile
])
def test_cut_batch_ranges_match_direct(kw):
    """The balanced planner's cut of a tile's batch keys (parts with last = their last row + 2, then one open part):
    the partial records of such parts, merged, equal the row-by-row call."""
    c = small_case(seed=24, H=4, Hkv=2, rows_per_tile=64, **kw)
    o = host.options_mi355x(64, 256)
    o.cut_batch, o.item_steps, o.part_steps, o.min_chunk, o.min_span, o.granule = 1, 1, 0, 32, 64, 32
    tiles, jobs, parts = host.plan_tiles(c.trees, c.params.Hkv, c.params.window, c.pos if c.params.window else None, o)
    assert any(int(x["last"]) >= 2 for x in tiles) and parts > 0
    got = ob.attn_tiles(c.params, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, tiles, c.trees, jobs, parts)
    assert max_abs(got, oracle_direct(c), c.params.dtype) <= 1e-3


def test_split_count_invariance_is_tight():
    c = small_case(seed=22, seqs=((2048, 1),))
    outs = []
    for groups in (2, 16, 64, 256, 4096):
        tiles, jobs, parts = _plan(c, 512, groups)
        outs.append(f32(ob.attn_tiles(c.params, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, tiles, c.trees,
                                      jobs, parts), c.params.dtype))
    for o in outs[1:]:
        assert np.abs(o - outs[0]).max() <= 5e-4   # fp32 regrouping, then one fp16 rounding


def test_window_at_least_context_equals_causal():
    a = small_case(seed=23, seqs=((77, 9),))
    b = small_case(seed=23, seqs=((77, 9),), window=77 + 9)
    assert (oracle_direct(a) == oracle_direct(b)).all()
    c = small_case(seed=23, seqs=((77, 9),), window=20)
    assert (oracle_direct(a) != oracle_direct(c)).any()


def test_single_row_verify_equals_decode():
    a = small_case(seed=24, seqs=((50, 1),))
    b = small_case(seed=24, seqs=((50, 1),), desc_fn=lambda M: synth.verify_desc(M, 1))
    assert (oracle_direct(a) == oracle_direct(b)).all()


def test_chunked_prefill_equals_one_pass_equals_decode_steps():
    """4 chunks against the growing cache == one causal pass == token-by-token decode."""
    p_ = dict(seed=25, H=4, Hkv=2, seqs=((0, 48),))
    whole = small_case(**p_)
    p = whole.params
    ref = f32(oracle_direct(whole), p.dtype)
    want = brute(whole)
    assert np.abs(ref - want).max() <= TOL
    # replay in chunks of 12 (and of 1): rows [s, s + n) with P = s cached via kv_save into a pool
    for chunk in (12, 1):
        pool = np.zeros(4 * 2 * p.bt * p.kv_ld, np.uint16)
        blocks = np.array([2, 0, 3, 1], np.int32)
        out = np.zeros_like(ref)
        for s in range(0, 48, chunk):
            trees = np.array([(s, s, 0, chunk)], abi.TREE_DT)
            pos = whole.pos.copy()
            o = ob.attn_direct(p, whole.Q, whole.Kb, whole.Vb, pool, blocks, np.zeros_like(whole.desc), pos, trees)
            out[s:s + chunk] = f32(o, p.dtype)[s:s + chunk]
            saves = np.array(ho.kv_saves(s, s, chunk, [int(b) for b in blocks], p.bt), abi.KVSAVE_DT)
            ob.kv_save(p, whole.Kb, whole.Vb, pool, saves)
        assert np.abs(out - ref).max() <= 1e-3


def test_page_permutation_is_bit_invariant():
    """Gathering is index work: permuting the pool's pages with the table permuted accordingly
    must not change one bit (tools/qsa_check.mm:120-123 shuffles its table for this)."""
    a = small_case(seed=26, seqs=((100, 2), (45, 1)), n_blocks=32)
    o1 = oracle_direct(a)
    rng = np.random.default_rng(99)
    perm = rng.permutation(a.n_blocks)           # new id of old block b is perm[b]
    blk2 = 2 * a.params.bt * a.params.kv_ld
    pool2 = np.zeros_like(a.pool_ref)
    for b in range(a.n_blocks):
        pool2[perm[b] * blk2:(perm[b] + 1) * blk2] = a.pool_ref[b * blk2:(b + 1) * blk2]
    o2 = ob.attn_direct(a.params, a.Q, a.Kb, a.Vb, pool2, perm[a.blocks].astype(np.int32), a.desc, a.pos, a.trees)
    assert (o1 == o2).all()
    # and the page walk alone
    K1, V1 = ob.kv_gather(a.params, a.pool_ref, a.blocks[:7], 100)
    K2, V2 = ob.kv_gather(a.params, pool2, perm[a.blocks[:7]].astype(np.int32), 100)
    assert (K1 == K2).all() and (V1 == V2).all()


def test_heads_of_a_group_with_equal_q_agree():
    c = small_case(seed=27, H=8, Hkv=2, seqs=((60, 2),))
    HD = c.params.head_dim
    for h in range(1, 4):
        c.Q[:, h * HD:(h + 1) * HD] = c.Q[:, :HD]
    o = oracle_direct(c)
    for h in range(1, 4):
        assert (o[:, h * HD:(h + 1) * HD] == o[:, :HD]).all()
    assert (o[:, 4 * HD:5 * HD] != o[:, :HD]).any()     # other KV head


def test_batch_key_equals_same_key_in_cache():
    """The `last` tile's batch keys behave as if appended to the cache."""
    a = small_case(seed=28, H=4, Hkv=2, seqs=((31, 1),))
    p = a.params
    o_batch = oracle_direct(a)
    pool = a.pool_ref.copy()
    saves = np.array(ho.kv_saves(0, 31, 1, [int(b) for b in a.blocks], p.bt), abi.KVSAVE_DT)
    ob.kv_save(p, a.Kb, a.Vb, pool, saves)
    trees = np.array([(0, 32, 0, 1)], abi.TREE_DT)
    desc = np.array([[1, 0, 0, 0]], np.int32)   # the row's own batch key hidden: only the cache
    o_cache = ob.attn_direct(p, a.Q, a.Kb, a.Vb, pool, a.blocks, desc, a.pos, trees)
    assert (o_batch == o_cache).all()


def test_kv_copy_blocks_copies_every_layer():
    p = synth.make_params(4, 2, 128, abi.ESP_F16, 16)
    region = 4 * 2 * p.bt * p.kv_ld
    rng = np.random.default_rng(3)
    pool = rng.integers(0, 65535, 3 * region).astype(np.uint16)
    before = pool.copy()
    ob.kv_copy_blocks(p, pool, [(1, 3), (0, 2)], 3, region)
    blk2 = 2 * p.bt * p.kv_ld
    for l in range(3):
        r = pool[l * region:(l + 1) * region].reshape(4, blk2)
        b = before[l * region:(l + 1) * region].reshape(4, blk2)
        assert (r[3] == b[1]).all() and (r[2] == b[0]).all() and (r[:2] == b[:2]).all()


def test_noncausal_root_is_full_bidirectional_attention(oracle):
    """anc_len = root_len on every row (the reference's noncausal roots, src/model/impl/forest.h:2402-2403, mask rule
    kernels/40_attention.metal:104-113): row i sees every row of the root, later ones included. Against a dense softmax
    in float64 that knows no masks at all, and against the truth table of the rule."""
    from espetero_amd import synth
    from helpers import max_abs, oracle_direct, small_case
    M = 7
    c = small_case(seed=91, H=4, Hkv=2, seqs=((0, M),), rows_per_tile=8, desc_fn=lambda m: np.tile(np.array([0, 0, m, 0], np.int32), (m, 1)))
    vis = oracle.visible_mask(c.params, c.trees[0], c.desc, c.pos)
    assert vis.shape == (M, M) and vis.all()
    p = c.params
    q = oracle.to_f32(c.Q, p.dtype).astype(np.float64).reshape(M, p.H, p.head_dim)
    k = oracle.to_f32(c.Kb, p.dtype).astype(np.float64).reshape(M, p.Hkv, p.head_dim)
    v = oracle.to_f32(c.Vb, p.dtype).astype(np.float64).reshape(M, p.Hkv, p.head_dim)
    want = np.zeros((M, p.H, p.head_dim))
    for h in range(p.H):
        s = q[:, h] @ k[:, h // 2].T * p.scale
        w = np.exp(s - s.max(axis=1, keepdims=True))
        want[:, h] = (w / w.sum(axis=1, keepdims=True)) @ v[:, h // 2]
    assert max_abs(oracle_direct(c), want.reshape(M, -1), p.dtype) <= 2e-3
    # with a cache in front: the cached keys and the whole root
    c = small_case(seed=92, H=4, Hkv=2, seqs=((37, M),), rows_per_tile=8, desc_fn=lambda m: np.tile(np.array([0, 0, m, 0], np.int32), (m, 1)))
    assert oracle.visible_mask(c.params, c.trees[0], c.desc, c.pos).all()
