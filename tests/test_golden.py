"""The CPU checker and the host planner against the committed fixtures of tests/golden/ (made by
tests/golden/make_fixtures.py from float64 formulas that share no code with the checker). The reference
holds no vectors for this path, so these are this repository's own; what they pin is that the checker
keeps agreeing with the dense float64 statement of the semantics, whatever is changed later."""
import json
import os

import numpy as np
import pytest

from espetero_amd import abi, host
from oracle import binding as ob

from helpers import GOLDEN, beyond_rounding, golden_names, load_golden_attention, tol_for


def test_the_fixture_set_is_complete():
    assert len(golden_names("attention")) == 12 and golden_names("prep") == ["gemma", "gemma512", "omni", "qwen35"]
    assert os.path.exists(os.path.join(GOLDEN, "gate.npz")) and os.path.exists(os.path.join(GOLDEN, "planner.json"))


@pytest.mark.parametrize("name", golden_names("attention"))
def test_checker_direct_and_tiled_forms_match_the_fixture(name):
    c, want = load_golden_attention(name)
    p = c.params
    got = ob.to_f32(ob.attn_direct(p, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees), p.dtype)
    assert beyond_rounding(got.reshape(want.shape), want, p.dtype, False) <= tol_for(p.dtype, unrounded=True)
    # the same through tiles, partial records and the merge, planned by the reference's rule and by the balanced one
    for o in (host.options_reference(), host.options_mi355x(p.rows_per_tile, 64)):
        rows = p.rows_per_tile
        p.rows_per_tile = o.rows_per_tile
        tiles, jobs, n_parts = host.plan_tiles(c.trees, p.Hkv, p.window, c.pos if p.window else None, o)
        got = ob.to_f32(ob.attn_tiles(p, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, tiles, c.trees, jobs, n_parts), p.dtype)
        p.rows_per_tile = rows
        assert beyond_rounding(got.reshape(want.shape), want, p.dtype, False) <= tol_for(p.dtype, unrounded=True), (name, o.rows_per_tile)


@pytest.mark.parametrize("kind", golden_names("prep"))
def test_checker_prep_matches_the_fixture(kind):
    z = np.load(os.path.join(GOLDEN, f"prep_{kind}.npz"), allow_pickle=False)
    p = abi.PrepParams()
    for k, v in json.loads(str(z["meta"])).items():
        setattr(p, k, v)
    sel = z["rope_sel"] if z["rope_sel"].size else None
    n = z["X"].shape[0]
    got = ob.attn_prep(p, z["X"], z["qn_w"], z["kn_w"], z["pos"], z["inv_freq"], sel, n)
    half_ulp = 2.0 ** -11 if p.dtype == abi.ESP_F16 else 2.0 ** -8
    for g, w in zip(got, (z["Q"], z["K"], z["V"])):
        g = ob.to_f32(g, p.dtype).astype(np.float64)
        assert np.all(np.abs(g - w) <= 1.02 * half_ulp * np.abs(w) + 1e-6)


def test_checker_gate_matches_the_fixture():
    z = np.load(os.path.join(GOLDEN, "gate.npz"), allow_pickle=False)
    p = abi.GateParams()
    for k, v in json.loads(str(z["meta"])).items():
        setattr(p, k, v)
    n = z["X"].shape[0]
    got, dots = ob.head_gate(p, z["O_in"], z["X"], z["Wg"], n, want_dots=True)
    assert np.abs(dots - z["dots"]).max() <= 1e-4
    assert np.abs(ob.to_f32(got, p.dtype)[:, :p.H * p.head_dim] - z["O"]).max() <= 1e-3


def test_host_planner_reference_rule_matches_the_fixture():
    """The C++ planner under the reference's options on the benchmark shapes == the recorded plan."""
    plans = json.load(open(os.path.join(GOLDEN, "planner.json")))
    assert sorted(plans) == ["c1", "c2", "c3_p6144", "c4_decode_global", "c5"]
    for name, w in plans.items():
        trees = np.array([tuple(t) for t in w["trees"]], abi.TREE_DT)
        tiles, jobs, n_parts = host.plan_tiles(trees, w["groups"], 0, None, host.options_reference())
        as_list = lambda r: [int(x) for x in r.tolist()]  # noqa: E731
        assert (len(tiles), len(jobs), n_parts) == (w["n_tiles"], w["n_jobs"], w["n_parts"]), name
        assert as_list(tiles[0]) == w["first_tile"] and as_list(tiles[-1]) == w["last_tile"], name
        if w["first_job"] is not None:
            assert as_list(jobs[0]) == w["first_job"], name
        t32 = tiles.view(np.int32).reshape(-1, 8).astype(np.int64)
        assert [int(x) for x in t32.sum(axis=0)] == w["tile_sum"], name
