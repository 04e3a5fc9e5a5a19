"""The HIP path, through the C ABI, against the committed fixtures of tests/golden/ (float64 expected
outputs; tests/golden/make_fixtures.py). Bar: max-abs 2e-3 for the attention, after half a unit in the last place of a bf16
output (helpers.beyond_rounding); one unit in the last place of the storage type for the prep and the gate."""
import json
import os

import numpy as np
import pytest
import torch

from espetero_amd import abi, device, host
from oracle import binding as ob

from helpers import GOLDEN, beyond_rounding, golden_names, load_golden_attention, tol_for

pytestmark = pytest.mark.gpu


def _dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("name", golden_names("attention"))
def test_attention_matches_the_fixture(name):
    from gpu_utils import run_case
    c, want = load_golden_attention(name)
    print(f"golden attention {name}", flush=True)
    got = ob.to_f32(run_case(c), c.params.dtype)
    assert beyond_rounding(got, want, c.params.dtype, False) <= tol_for(c.params.dtype, unrounded=True)
    if c.params.rows_per_tile * (c.params.H // c.params.Hkv) <= 32:   # also as the largest tiles of the tiled kernel
        rows = device.plan_hint3(c.params)[2]
        c.params.rows_per_tile = rows
        got = ob.to_f32(run_case(c, host.options_mi355x(rows, 8)), c.params.dtype)
        assert beyond_rounding(got, want, c.params.dtype, False) <= tol_for(c.params.dtype, unrounded=True)


@pytest.mark.parametrize("kind", golden_names("prep"))
def test_prep_matches_the_fixture(kind):
    device.init(0)
    z = np.load(os.path.join(GOLDEN, f"prep_{kind}.npz"), allow_pickle=False)
    p = abi.PrepParams()
    for k, v in json.loads(str(z["meta"])).items():
        setattr(p, k, v)
    n = z["X"].shape[0]
    tdt = torch.float16 if p.dtype == abi.ESP_F16 else torch.bfloat16
    Q = torch.zeros(n, p.q_ld, dtype=tdt, device="cuda")
    Kb = torch.zeros(n, p.kv_ld, dtype=tdt, device="cuda")
    Vb = torch.zeros_like(Kb)
    sel = _dev(z["rope_sel"]) if z["rope_sel"].size else None
    device.attn_prep(p, _dev(z["X"]), _dev(z["qn_w"]), _dev(z["kn_w"]), _dev(z["pos"]), _dev(z["inv_freq"]), sel, Q, Kb, Vb, None, None, n)
    torch.cuda.synchronize()
    ulp = 2.0 ** -10 if p.dtype == abi.ESP_F16 else 2.0 ** -7      # one unit in the last place, relative
    for g, w in zip((Q, Kb, Vb), (z["Q"], z["K"], z["V"])):
        g = g.float().cpu().numpy().astype(np.float64)
        assert np.all(np.abs(g - w) <= 1.02 * ulp * np.abs(w) + 1e-6)


def test_gate_matches_the_fixture():
    device.init(0)
    z = np.load(os.path.join(GOLDEN, "gate.npz"), allow_pickle=False)
    p = abi.GateParams()
    for k, v in json.loads(str(z["meta"])).items():
        setattr(p, k, v)
    n = z["X"].shape[0]
    O = _dev(z["O_in"].view(np.int16))
    dots = torch.zeros(n, p.H, dtype=torch.float32, device="cuda")
    device.head_gate(p, O, _dev(z["X"].view(np.int16)), _dev(z["Wg"].view(np.int16)), dots, n)
    torch.cuda.synchronize()
    assert np.abs(dots.cpu().numpy() - z["dots"]).max() <= 1e-4
    got = ob.to_f32(O.cpu().numpy().view(np.uint16), p.dtype)[:, :p.H * p.head_dim]
    assert np.abs(got - z["O"]).max() <= 1e-3
