"""Parity of the HIP path with the CPU checker, through the C ABI, on a real MI355X.

Bar: max-abs 2e-3 at fp32 accumulation, the tolerance the path's contract states, on the difference that is left
once the rounding of the stored output itself is taken off (helpers.max_abs: nothing on fp16; on bf16 half a unit
in the last place against an unrounded expectation, one unit against the checker's own bf16 output). Seeded inputs,
sizes the checker finishes in seconds; the full benchmark sizes are covered by
size-independent properties in test_gpu_properties.py.
"""
import numpy as np
import pytest

from espetero_amd import abi, host, synth

from helpers import brute, f32, max_abs, oracle_direct, sharp_case, small_case, tol_for

pytestmark = pytest.mark.gpu


def _check(case, options=None, **kw):
    from gpu_utils import run_case
    print(f"case {case.name} seqs={case.meta['seqs']} R={case.params.rows_per_tile}", flush=True)
    got = run_case(case, options, **kw)
    want = oracle_direct(case, threads=8)
    err = max_abs(got, want, case.params.dtype)
    assert err <= tol_for(case.params.dtype), f"{case.name}: max abs {err}"
    return got


# ---- streaming kernel: decode and verify shapes
@pytest.mark.parametrize("kw", [
    dict(seqs=((70, 1), (33, 1)), rows_per_tile=1),                     # ragged page tails
    dict(seqs=((1, 1), (0, 1), (16, 1), (31, 1), (32, 1)), rows_per_tile=1),  # empty and tiny caches
    dict(seqs=((1000, 1), (17, 1), (5000, 1)), rows_per_tile=1),        # split + unsplit mixed
    dict(seqs=((300, 1),), H=8, Hkv=8, rows_per_tile=1),                # G = 1
    dict(seqs=((300, 1),), H=12, Hkv=2, rows_per_tile=1),               # G = 6
    dict(seqs=((300, 1),), H=10, Hkv=2, rows_per_tile=1, dtype=abi.ESP_BF16),  # G = 5, bf16
    dict(seqs=((777, 1), (100, 1)), H=4, Hkv=2, HD=256, rows_per_tile=1),      # head_dim 256
    dict(seqs=((200, 1),), bt=64, rows_per_tile=1),                     # the reference's block size
    dict(seqs=((1030, 4), (90, 4)), rows_per_tile=4, desc_fn=lambda M: synth.verify_desc(M, 1)),   # verify
    dict(seqs=((500, 3),), H=16, Hkv=2, rows_per_tile=4, desc_fn=lambda M: synth.verify_desc(M, 2)),  # 2 roots + 1
    dict(seqs=((400, 6), (64, 2)), H=4, Hkv=2, rows_per_tile=8),        # short causal chunks on the streaming kernel
    dict(seqs=((900, 1), (40, 1)), window=128, rows_per_tile=1),        # sliding window over block lists
    dict(seqs=((900, 1), (2000, 1)), window=256, ring_layer=True, rows_per_tile=1),  # sliding window over rings
    dict(seqs=((300, 5),), window=64, rows_per_tile=8, H=4, Hkv=2),     # window on multi-row tiles
    dict(seqs=((200, 8),), rows_per_tile=8, H=4, Hkv=2, bidi=1, desc_fn=lambda M: synth.image_desc(M, 2, 6)),  # bidirectional span
])
def test_stream_kernel_matches_checker(kw):
    _check(small_case(seed=31, fill_unused=not kw.get("ring_layer", False), **kw))


# ---- head dim 512 (Gemma 4's full-attention layers): wavefront pairs share a unit
@pytest.mark.parametrize("kw", [
    dict(seqs=((777, 1), (100, 1)), H=8, Hkv=1, rows_per_tile=1),                   # G = 8 decode
    dict(seqs=((1, 1), (0, 1), (16, 1), (31, 1), (32, 1), (33, 1)), H=16, Hkv=2, rows_per_tile=1),  # 0, 1, 2, 3 units
    dict(seqs=((5000, 1), (17, 1)), H=16, Hkv=2, rows_per_tile=1),                  # split + merge
    dict(seqs=((300, 2), (45, 1)), H=8, Hkv=2, rows_per_tile=2, dtype=abi.ESP_BF16),  # G = 4, two rows, bf16
    dict(seqs=((260, 2),), H=8, Hkv=1, rows_per_tile=2, desc_fn=lambda M: synth.verify_desc(M, 1)),  # 16 packed rows
    dict(seqs=((200, 1),), H=4, Hkv=2, bt=64, rows_per_tile=1),                     # the reference's block size
    dict(seqs=((900, 1), (40, 1)), H=4, Hkv=1, window=128, rows_per_tile=1),        # window (not a Gemma shape; same code)
    dict(seqs=((90, 7),), H=4, Hkv=2, rows_per_tile=8),                             # G = 2, 8-row tiles: batch keys
    dict(seqs=((700, 4), (33, 4)), H=8, Hkv=1, rows_per_tile=2, desc_fn=lambda M: synth.verify_desc(M, 1)),  # a 4-row verify tree as two 2-row tiles
    # 32 packed rows: two wavefront pairs of one workgroup, one column tile each, walking the same units
    dict(seqs=((700, 4), (33, 4), (0, 3)), H=8, Hkv=1, rows_per_tile=4, desc_fn=lambda M: synth.verify_desc(M, 1)),  # a 4-row verify tree in one pass
    dict(seqs=((5000, 4), (900, 2)), H=16, Hkv=2, rows_per_tile=4, dtype=abi.ESP_BF16),                # split + merge, ragged last tile, bf16
    dict(seqs=((300, 1), (77, 1)), H=32, Hkv=1, rows_per_tile=1),                                        # G = 32
    dict(seqs=((900, 7), (40, 3)), H=12, Hkv=3, window=128, rows_per_tile=8),                           # G = 4, 8-row tiles: the pairs hold different rows under a window
    dict(seqs=((900, 4), (2000, 4)), H=8, Hkv=1, window=256, ring_layer=True, rows_per_tile=4, desc_fn=lambda M: synth.verify_desc(M, 2)),
    dict(seqs=((200, 8),), H=4, Hkv=1, rows_per_tile=8, bt=64, bidi=1, desc_fn=lambda M: synth.image_desc(M, 2, 6)),   # image span across the two pairs' rows
])
def test_stream_kernel_head_dim_512(kw):
    _check(small_case(seed=37, HD=512, fill_unused=True, **kw))


@pytest.mark.parametrize("P,bt", [(10, 32), (15, 32), (74, 32), (26, 64), (15, 16)])
def test_stream_kernel_partial_unit_at_head_dim_256(P, bt):
    """A short cache whose keys all sit in one partial 16-key unit: every score counts. (The fourth register of
    that unit's score tile was once read before the last matrix instruction had written it: keys 3, 7, 11
    came out with the weight of a dot product short of its last 32 dims, 4e-2 off at P = 10.)"""
    c = small_case(seed=38, H=2, Hkv=1, HD=256, bt=bt, seqs=((P, 1),), rows_per_tile=1, fill_unused=True)
    _check(c)
    c = small_case(seed=39, H=16, Hkv=1, HD=256, bt=bt, seqs=((P, 1), (P + 3, 1)), rows_per_tile=1, dtype=abi.ESP_BF16)
    _check(c)


def test_stream_kernel_reference_planner_records():
    """The kernels accept the reference planner's own records (8-row tiles, 32-key chunks)."""
    c = small_case(seed=32, seqs=((1024, 1),), H=32, Hkv=4, rows_per_tile=8)
    _check(c, host.options_reference())


def test_stream_kernel_without_desc_is_plain_causal():
    c = small_case(seed=33, seqs=((100, 3),), rows_per_tile=4)
    _check(c, with_desc=False)


def test_stream_kernel_split_invariance():
    from gpu_utils import run_case
    c = small_case(seed=34, seqs=((4096, 1), (333, 1)), H=32, Hkv=4, rows_per_tile=1)
    outs = [f32(run_case(c, host.options_mi355x(1, wg)), c.params.dtype) for wg in (8, 64, 512, 4096)]
    for o in outs[1:]:
        assert np.abs(o - outs[0]).max() <= 1e-3


def test_stream_kernel_is_deterministic():
    from gpu_utils import run_case
    c = small_case(seed=35, seqs=((3000, 1), (2000, 2)), H=32, Hkv=4, rows_per_tile=2)
    a = run_case(c)
    for _ in range(3):
        assert (run_case(c) == a).all()


@pytest.mark.parametrize("kw,wg", [
    (dict(seqs=((4096, 1), (333, 1), (2000, 1)), H=32, Hkv=4, rows_per_tile=1), 256),          # decode, G = 8
    (dict(seqs=((3000, 4), (1500, 3)), H=32, Hkv=4, rows_per_tile=4, desc_fn=lambda M: synth.verify_desc(M, 1)), 128),  # two column tiles
    (dict(seqs=((2500, 1), (700, 1)), H=4, Hkv=2, HD=256, rows_per_tile=1, dtype=abi.ESP_BF16), 64),
    (dict(seqs=((5000, 1), (900, 1)), H=16, Hkv=2, HD=512, rows_per_tile=1), 64),               # wavefront pairs
    (dict(seqs=tuple((200 + 37 * i, 1) for i in range(70)), H=8, Hkv=2, rows_per_tile=1), 2048),  # more jobs than one wavefront looks up at once
    (dict(seqs=((900, 1), (2000, 1)), window=256, ring_layer=True, rows_per_tile=1), 64),
])
def test_stream_kernel_merge_as_its_own_call_gives_the_same_bits(kw, wg):
    """esp_attn_forward with n_jobs = 0 followed by esp_attn_combine gives the bits of the one call that
    does both, run after run, and both are the checker's result."""
    from gpu_utils import plan, run_case
    c = small_case(seed=47, fill_unused=not kw.get("ring_layer", False), **kw)
    opts = host.options_mi355x(c.params.rows_per_tile, wg)
    tiles, jobs, n_parts = plan(c, opts)
    assert len(jobs) >= 2 and n_parts > len(jobs), "the plan must split"
    print(f"case seqs={c.meta['seqs'][:4]} tiles={len(tiles)} jobs={len(jobs)} parts={n_parts}", flush=True)
    two = run_case(c, opts, two_step=True)
    for _ in range(3):
        assert (run_case(c, opts) == two).all()
    assert max_abs(two, oracle_direct(c, threads=8), c.params.dtype) <= tol_for(c.params.dtype)


def test_gate():
    import torch
    from gpu_utils import run_case
    c = small_case(seed=36, seqs=((200, 1), (50, 1)), rows_per_tile=1)
    p = c.params
    g = np.random.default_rng(0).standard_normal((c.n_rows, p.H, 2 * p.head_dim)).astype(np.float32)
    gd = torch.from_numpy(g).cuda()
    p.gate = gd.data_ptr()
    p.gate_ld, p.gate_hs, p.gate_off = p.H * 2 * p.head_dim, 2 * p.head_dim, p.head_dim
    got = f32(run_case(c), p.dtype)
    p.gate = None
    want = brute(c) / (1.0 + np.exp(-g[:, :, p.head_dim:].reshape(c.n_rows, -1).astype(np.float64)))
    assert np.abs(got - want).max() <= 2e-3


# ---- tiled MFMA kernel: prefill shapes
@pytest.mark.parametrize("kw", [
    dict(seqs=((0, 200),)),                                             # first chunk: batch keys only
    dict(seqs=((300, 130), (17, 5)), fill_unused=True),                 # chunk against a cache, ragged
    dict(seqs=((64, 256),), H=10, Hkv=2, dtype=abi.ESP_BF16),           # GQA 5, bf16 (prefill benchmark shape)
    dict(seqs=((100, 140),), H=4, Hkv=2, HD=256),                       # head_dim 256
    dict(seqs=((500, 200),), window=128, H=4, Hkv=2),                   # sliding window
    dict(seqs=((700, 150),), window=256, ring_layer=True, H=4, Hkv=2),  # sliding window, rings
    dict(seqs=((90, 40),), desc_fn=lambda M: synth.verify_desc(M, 30), H=4, Hkv=2),  # wide verify tree
    dict(seqs=((128, 128),), bt=64, H=4, Hkv=2),
    dict(seqs=((100, 140),), H=4, Hkv=2, bidi=1, desc_fn=lambda M: synth.image_desc(M, 10, 90)),   # bidirectional span
    dict(seqs=((1500, 130),), H=4, Hkv=2, HD=256),                      # long cached range: the mask-free loop, head_dim 256
    dict(seqs=((1203, 128), (700, 40)), bt=64, H=4, Hkv=2, fill_unused=True),  # the same at the reference's block size, ragged end
])
def test_tiled_kernel_matches_checker(kw):
    _check(small_case(seed=41, rows_per_tile=128, **kw))


# ---- logits of several units, a row maximum that keeps moving
@pytest.mark.parametrize("dtype", [abi.ESP_F16, abi.ESP_BF16])
@pytest.mark.parametrize("kw", [
    dict(seqs=((700, 130),)),                          # the cached run: the reference moves in first and second half steps alike
    dict(seqs=((0, 400),)),                            # the batch run only
    dict(seqs=((40, 300), (333, 70))),                 # a cached range that ends inside a half step, then batch rows
    dict(seqs=((1000, 140),), HD=256, H=4),            # head dim 256: the lazily moved maximum
    dict(seqs=((600, 70),), HD=512, H=4, rows_per_tile=64),
    dict(seqs=((900, 1), (77, 1)), H=16, rows_per_tile=1),                                          # streaming kernel, decode
    dict(seqs=((500, 4),), H=16, rows_per_tile=4, desc_fn=lambda M: synth.verify_desc(M, 1)),     # and verify
])
def test_sharp_softmax_with_a_moving_maximum(kw, dtype):
    """Scores with a spread of 8 nats (fp16; 4.5 on bf16) whose maximum grows along the keys: the tiled kernel's head-dim-128 path
    takes no per-step maximum and must notice by itself when the row's reference has to move (mid-row rescale of
    the accumulators, also deferred past the first half step's P V); every kernel must keep the scale out of
    the operands' rounding. Bar: 2e-3 against the float64 brute force, the stored output's own rounding excepted,
    on both element types; the checker is held to the same bar on the same case."""
    from gpu_utils import run_case
    # bf16 keeps 8 bits of every probability: at a spread of 8 nats that rounding alone reaches the bar (the
    # checker itself reads 2.0e-3 there), so bf16 runs at a spread of 4.5 nats, where it leaves a margin.
    spread = dict(sigma_q=2.0, k_hi=4.0) if dtype == abi.ESP_F16 else dict(sigma_q=1.5, k_hi=3.0)
    c = sharp_case(51, dtype, **spread, **kw)
    print(f"case sharp seqs={c.meta['seqs']} HD={c.params.head_dim} dtype={dtype}", flush=True)
    want = brute(c)
    err_checker = max_abs(oracle_direct(c, threads=8), want, dtype)
    err = max_abs(run_case(c), want, dtype)
    print(f"  max abs beyond rounding: kernel {err:.2e}, checker {err_checker:.2e}", flush=True)
    assert err_checker <= 2e-3
    assert err <= 2e-3


# ---- head dim 512 prefill: 64-row tiles, wavefront pairs split the dims
@pytest.mark.parametrize("kw", [
    dict(seqs=((0, 200),), H=4, Hkv=2),                                 # first chunk: batch keys only
    dict(seqs=((300, 130), (17, 5)), H=4, Hkv=2, fill_unused=True),     # chunk against a cache, ragged
    dict(seqs=((64, 150),), H=16, Hkv=2, dtype=abi.ESP_BF16),           # G = 8 (Gemma 4's grouping), bf16
    dict(seqs=((500, 100),), window=128, H=2, Hkv=1),                   # sliding window (not a Gemma shape; same code)
    dict(seqs=((700, 70),), window=256, ring_layer=True, H=2, Hkv=1),   # rings
    dict(seqs=((90, 40),), desc_fn=lambda M: synth.verify_desc(M, 30), H=4, Hkv=2),  # wide verify tree
    dict(seqs=((128, 128),), bt=64, H=4, Hkv=2),
    dict(seqs=((100, 140),), H=2, Hkv=1, bidi=1, desc_fn=lambda M: synth.image_desc(M, 10, 90)),   # bidirectional span
    dict(seqs=((1203, 64), (700, 40)), bt=64, H=4, Hkv=2, fill_unused=True),  # long cached ranges, ragged end
    dict(seqs=((100, 2), (33, 1)), H=32, Hkv=1, rows_per_tile=2),       # G = 32, two rows: more packed rows (64) than the streaming kernel takes
    dict(seqs=((150, 20),), H=4, Hkv=2, rows_per_tile=24),              # tiles smaller than the kernel's 64 rows
    dict(seqs=((4127, 96),), H=2, Hkv=1),                               # 258 cached sub-blocks, the last one partial: the mask-free iterations, 64 addresses at a time
    dict(seqs=((2072, 70), (95, 3)), bt=32, H=4, Hkv=2, dtype=abi.ESP_BF16, fill_unused=True),   # the same beside a tile with too few for any
])
def test_tiled_kernel_head_dim_512(kw):
    _check(small_case(seed=44, HD=512, **{"rows_per_tile": 64, **kw}))


def test_tiled_kernel_head_dim_512_split_and_gate():
    """Split tiles merged by the combine kernel at head dim 512, with a head-wise gate in the epilogue."""
    import torch
    from gpu_utils import run_case
    c = small_case(seed=45, HD=512, seqs=((2000, 70),), H=4, Hkv=2, rows_per_tile=64)
    _check(c, host.options_mi355x(64, 64))
    p = c.params
    g = np.random.default_rng(1).standard_normal((c.n_rows, p.H)).astype(np.float32)
    gd = torch.from_numpy(g).cuda()
    p.gate, p.gate_ld, p.gate_hs, p.gate_off, p.gate_headwise = gd.data_ptr(), p.H, 1, 0, 1
    split = f32(run_case(c, host.options_mi355x(64, 64)), p.dtype)
    whole = f32(run_case(c, host.options_mi355x(64, 1)), p.dtype)
    p.gate, p.gate_headwise = None, 0
    want = brute(c).reshape(c.n_rows, p.H, -1) / (1.0 + np.exp(-g.astype(np.float64)))[:, :, None]
    assert np.abs(split - want.reshape(c.n_rows, -1)).max() <= 2e-3
    assert np.abs(whole - want.reshape(c.n_rows, -1)).max() <= 2e-3


@pytest.mark.parametrize("HD,rows", [(128, 32), (256, 32), (256, 128), (512, 64)])
def test_tiled_kernel_one_row_remainder_tile_on_a_windowed_layer(HD, rows):
    """A chunk of k * rows + 1 rows on a sliding layer: the last tile is one row, its first batch sub-block
    starts below the window's lower edge, and no other row's position test covers those keys. (They once
    counted as visible: 0.18 off on that row.)"""
    for window, ring in ((17, False), (17, True), (40, False)):
        _check(small_case(seed=46, H=6, Hkv=3, HD=HD, bt=64, seqs=((565, 2 * rows + 3), (300, rows + 1)), rows_per_tile=rows,
                          window=window, ring_layer=ring, fill_unused=not ring))


@pytest.mark.parametrize("HD,rows,dtype", [(128, 128, abi.ESP_F16), (128, 64, abi.ESP_BF16), (256, 128, abi.ESP_BF16),
                                           (256, 32, abi.ESP_F16), (512, 64, abi.ESP_F16)])
@pytest.mark.parametrize("positions", ["consecutive", "pairs", "step_back"])
def test_tiled_kernel_chunk_longer_than_the_window(HD, rows, dtype, positions):
    """A chunk several windows long: most tiles' batch keys straddle the window's lower edge. Positions that rise by
    one per row take the window as a bound in row numbers; positions that repeat (two rows per position) or step
    back in the middle of the chunk take the per-key position test. The split target also cuts the cached range."""
    from gpu_utils import run_case
    window = 200
    c = small_case(seed=47, H=6, Hkv=3, HD=HD, bt=32, dtype=dtype, seqs=((333, 700), (50, 290), (0, 450)), rows_per_tile=rows,
                   window=window)
    if positions != "consecutive":
        for t in c.trees:
            P, M, base = int(t["P"]), int(t["M"]), int(t["base"])
            j = np.arange(M)
            c.pos[base:base + M, 0:3] = (P + (j // 2 if positions == "pairs" else np.where(j < M // 2, j, j - 37)))[:, None]
    _check(c, host.options_mi355x(rows, 64))
    if HD != 512 and positions == "consecutive":   # the same chunk with its rows read from the pool
        from test_gpu_rows_in_pool import pool_case
        pc = pool_case(seed=48, H=6, Hkv=3, HD=HD, bt=32, dtype=dtype, seqs=((320, 700), (60, 450)), rows_per_tile=rows, window=window)
        print(f"rows in pool: {pc.meta['seqs']}", flush=True)
        got = run_case(pc, host.options_mi355x(rows, 64), rows_in_pool=True)
        err = max_abs(got, oracle_direct(pc, threads=8), dtype)
        assert err <= tol_for(dtype), f"rows in pool: max abs {err}"


@pytest.mark.parametrize("kw", [
    dict(seqs=((0, 1500),), H=4, Hkv=2, dtype=abi.ESP_BF16),                        # a first chunk: batch keys only, ragged end
    dict(seqs=((130, 1100), (0, 700)), H=4, Hkv=2, HD=256),                         # a part that ends the cached keys and begins the batch keys
    dict(seqs=((0, 1400),), H=4, Hkv=2, HD=256, window=300, dtype=abi.ESP_BF16),    # cuts on both sides of the window's lower edge
    dict(seqs=((40, 1300),), H=2, Hkv=2, bt=64, bidi=1, desc_fn=lambda M: synth.image_desc(M, 500, 900)),   # rows that see beyond their own tile
    dict(seqs=((0, 1200),), H=2, Hkv=1, HD=512, rows_per_tile=64),                  # head dim 512
    dict(seqs=((16, 1400),), H=4, Hkv=2, rows_in_pool=True),                        # the rows read from the pool
    # a second tree whose rows begin 4 rows into a group of 16: a cut at a multiple of 64 of its own rows then falls inside a
    # staged sub-block, whose keys behind the cut belong to the next part (a random sweep found them counted twice by the
    # rows far enough below: the whole-half-step shortcut did not look at where the part's batch range ends)
    dict(seqs=((634, 244), (1295, 369)), H=32, Hkv=2, HD=256, dtype=abi.ESP_BF16, fill_unused=True, wg=5000),
    dict(seqs=((0, 250), (100, 900)), H=4, Hkv=2, dtype=abi.ESP_BF16, wg=5000),
])
def test_tiled_kernel_cuts_the_batch_keys_of_a_tile(kw):
    """With cut_batch the balanced rule cuts a tile's batch keys like its cached keys (a part whose batch range ends
    early carries last = its last row + 2). Switched on here, with a cost model without fixed costs so that it cuts;
    held to the checker, and to the uncut plan within the merge's own rounding."""
    from gpu_utils import plan, run_case
    in_pool = kw.pop("rows_in_pool", False)
    R, wg = kw.pop("rows_per_tile", 128), kw.pop("wg", 256)
    if in_pool:
        from test_gpu_rows_in_pool import pool_case
        c = pool_case(49, rows_per_tile=R, **kw)
    else:
        c = small_case(seed=49, rows_per_tile=R, **kw)
    o = host.options_mi355x(R, wg)
    o.cut_batch, o.item_steps, o.part_steps, o.min_chunk, o.min_span = 1, 1, 0, 128, 256
    tiles, _, n_parts = plan(c, o)
    cut = [x for x in tiles if int(x["last"]) >= 2]
    assert cut and n_parts > 0, "the plan has no part with a cut batch range"
    print(f"case seqs={c.meta['seqs']} R={R}: {len(tiles)} records, {len(cut)} with a cut batch range", flush=True)
    got = run_case(c, o, rows_in_pool=in_pool)
    err = max_abs(got, oracle_direct(c, threads=8), c.params.dtype)
    assert err <= tol_for(c.params.dtype), f"max abs {err}"
    whole = run_case(c, None, rows_in_pool=in_pool)
    assert np.abs(f32(got, c.params.dtype) - f32(whole, c.params.dtype)).max() <= 2e-3


def test_tiled_kernel_split_tiles_and_combine():
    """A single long-context tile group is split over key ranges and merged."""
    c = small_case(seed=42, seqs=((3000, 100),), H=4, Hkv=2, rows_per_tile=128)
    _check(c, host.options_mi355x(128, 64))


def test_chunked_prefill_then_decode_through_kv_save():
    """Chunks appended with esp_kv_save are what later chunks and decode steps read."""
    import torch
    from espetero_amd import device
    from gpu_utils import dev_u16, to_host_u16
    from oracle import host_oracle as ho
    whole = small_case(seed=43, H=8, Hkv=2, seqs=((0, 300),), rows_per_tile=128)
    p = whole.params
    want = f32(oracle_direct(whole, threads=8), p.dtype)
    device.init(0)
    n_blocks = 32
    pool = torch.zeros(n_blocks * 2 * p.bt * p.kv_ld, dtype=torch.int16, device="cuda")
    blocks = np.random.default_rng(1).permutation(n_blocks).astype(np.int32)[:20]
    Q, Kb, Vb = dev_u16(whole.Q), dev_u16(whole.Kb), dev_u16(whole.Vb)
    O = torch.zeros_like(Q)
    s = 0
    for n in (128, 100, 71, 1):     # three prefill chunks, then one decode step
        p.rows_per_tile = 128 if n > 1 else 1
        trees = np.array([(s, s, 0, n)], abi.TREE_DT)
        resident, groups = device.plan_hint(p)
        opts = host.options_mi355x(p.rows_per_tile, resident)
        tiles, jobs, n_parts = host.plan_tiles(trees, groups, 0, None, opts)
        dp = device.DevicePass(p, trees, tiles, jobs, n_parts, 300, blocks, None, None)
        dp.run(Q, Kb, Vb, pool, O)
        saves = np.array(ho.kv_saves(s, s, n, [int(b) for b in blocks], p.bt), abi.KVSAVE_DT)
        device.kv_save(p, Kb, Vb, pool, device.to_dev(saves), len(saves))
        torch.cuda.synchronize()
        s += n
    got = f32(to_host_u16(O).reshape(300, -1), p.dtype)
    assert np.abs(got - want).max() <= 2e-3
