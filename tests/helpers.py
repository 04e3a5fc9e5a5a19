"""Shared by the tests: small case builders and comparisons."""
import numpy as np

from espetero_amd import abi, synth
from oracle import binding as ob

TOL = 2e-3  # max-abs contract of the path (fp32 accumulation, fp16 / bf16 storage)


def f32(bits, dtype):
    return ob.to_f32(bits, dtype)


def bf16_ulp(x):
    """One unit in the last place of a bf16 number of x's magnitude: 8 significant bits, 2^(floor(log2 |x|) - 7)."""
    ax = np.maximum(np.abs(np.asarray(x, np.float64)), 2.0 ** -126)
    return 2.0 ** (np.floor(np.log2(ax)) - 7)


def beyond_rounding(got, want, dtype, want_rounded):
    """Largest |got - want| once the rounding of the stored output itself is taken off: nothing for fp16 (half a unit
    in the last place of an output below 1 is 2.4e-4, inside the bar), and for bf16 half a unit in the last place
    against an unrounded expectation, a whole unit against one that was itself rounded to bf16 (two results a hair
    apart may round to neighbouring bf16 numbers)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64).reshape(np.shape(got))
    allow = 0.0 if dtype == abi.ESP_F16 else bf16_ulp(np.maximum(np.abs(got), np.abs(want))) * (1.0 if want_rounded else 0.5)
    return float(np.maximum(np.abs(got - want) - allow, 0.0).max())


def max_abs(a_bits, b, dtype):
    """a: storage bits; b: storage bits (plain max-abs difference) or a float array, an unrounded expectation (the
    difference beyond the output's own rounding)."""
    a = f32(a_bits, dtype).astype(np.float64)
    if b.dtype == np.uint16:
        return float(np.abs(a - f32(b, dtype).astype(np.float64)).max())
    return beyond_rounding(a, b, dtype, False)


def tol_for(dtype, unrounded=False):
    """The bar for max_abs. Against an unrounded (float64) expectation: the contract's 2e-3 for both types, the
    rounding of the stored output itself excepted. Against the checker's own output in the storage type: 2e-3 on fp16;
    on bf16 both sides round their probabilities and their output to 8 significant bits, each is within 2e-3 of the
    exact result, and the bar between the two is 4e-3. (The tests' outputs stay below 1, where a result that rounds
    to the neighbouring bf16 number differs by at most 3.9e-3; against an unrounded expectation no such cap is needed.)"""
    return TOL if unrounded or dtype == abi.ESP_F16 else 4e-3


def small_case(seed=0, H=8, Hkv=2, HD=128, dtype=abi.ESP_F16, bt=16, seqs=((70, 1), (33, 1)), **kw):
    return synth.make_case("small", seed, H, Hkv, HD, dtype, bt, list(seqs), **kw)


def oracle_direct(case, threads=4):
    c = case
    return ob.attn_direct(c.params, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees, n_threads=threads)


def brute(case):
    c = case
    H, HD = c.params.H, c.params.head_dim
    return ob.brute_force(c.params, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees).reshape(c.n_rows, H * HD)


GOLDEN = __import__("os").path.join(__import__("os").path.dirname(__import__("os").path.abspath(__file__)), "golden")


def golden_names(prefix):
    import os
    return sorted(f[len(prefix) + 1:-4] for f in os.listdir(GOLDEN) if f.startswith(prefix + "_") and f.endswith(".npz"))


def load_golden_attention(name):
    """A committed attention fixture as (Case, expected O float64 [n_rows][H * head_dim])."""
    import json
    import os
    z = np.load(os.path.join(GOLDEN, f"attention_{name}.npz"), allow_pickle=False)
    m = json.loads(str(z["meta"]))
    p = synth.make_params(m["H"], m["Hkv"], m["head_dim"], m["dtype"], m["bt"], window=m["window"], ring=m["ring"],
                          scale=m["scale"], rows_per_tile=m["rows_per_tile"], bidi=m["bidi"])
    trees = np.ascontiguousarray(z["trees"]).view(abi.TREE_DT).reshape(-1)
    seqs = [(int(t["P"]), int(t["M"])) for t in trees]
    case = synth.Case(name, p, z["Q"], z["Kb"], z["Vb"], z["pool_ref"], m["n_blocks"], z["blocks"], trees, z["desc"], z["pos"],
                      m["n_rows"], dict(seqs=seqs, seed=None))
    return case, z["O"]
