"""Shared by the tests: small case builders and comparisons."""
import numpy as np

from espetero_amd import abi, synth
from oracle import binding as ob

from oracle.binding import TOL, beyond_rounding, bf16_ulp  # noqa: E402,F401  (the bar lives with the checker: bench and smoke use it too)


def f32(bits, dtype):
    return ob.to_f32(bits, dtype)


def max_abs(a_bits, b, dtype):
    """The difference beyond the stored output's own rounding (beyond_rounding). a: storage bits; b: storage bits (an
    expectation that was itself rounded to the storage type) or a float array (an unrounded expectation)."""
    a = f32(a_bits, dtype).astype(np.float64)
    if b.dtype == np.uint16:
        return beyond_rounding(a, f32(b, dtype).astype(np.float64), dtype, True)
    return beyond_rounding(a, b, dtype, False)


def tol_for(dtype, unrounded=False):
    """The bar for max_abs: the contract's 2e-3 for both element types and both kinds of expectation; what differs
    between them is only how much of the stored output's own rounding max_abs takes off first."""
    return TOL


def small_case(seed=0, H=8, Hkv=2, HD=128, dtype=abi.ESP_F16, bt=16, seqs=((70, 1), (33, 1)), **kw):
    return synth.make_case("small", seed, H, Hkv, HD, dtype, bt, list(seqs), **kw)


def sharp_case(seed, dtype, seqs, H=10, Hkv=2, HD=128, bt=16, sigma_q=2.0, k_lo=0.5, k_hi=4.0, rows_per_tile=128, **kw):
    """A case whose softmax is far from uniform and whose row maximum keeps moving: queries N(0, 1) * sigma_q,
    the keys of each sequence N(0, 1) * a ramp from k_lo (oldest) to k_hi (newest), so the scaled score's spread
    grows to sigma_q * k_hi (8 nats = 11.5 log2 units by default) and later keys outscore earlier ones by more than
    the 8 log2 units a lazily moved reference tolerates. Values stay N(0, 1) * 0.5 so outputs stay below 1."""
    c = synth.make_case("sharp", seed, H, Hkv, HD, dtype, bt, list(seqs), rows_per_tile=rows_per_tile, sigma=0.5, **kw)
    rng = np.random.default_rng(seed + 1000)
    kvw = Hkv * HD
    c.Q[:] = synth._bits(rng.standard_normal(c.Q.shape, dtype=np.float32) * sigma_q, dtype)
    pv = c.pool_ref.reshape(c.n_blocks, 2, bt, kvw)
    for t in c.trees:
        P, M, base, tab = int(t["P"]), int(t["M"]), int(t["base"]), int(t["table"])
        n = P + M
        ramp = (k_lo + (k_hi - k_lo) * np.arange(n) / max(n - 1, 1)).astype(np.float32)[:, None]
        K = synth._bits(rng.standard_normal((n, kvw), dtype=np.float32) * ramp, dtype)
        for j in range(P):
            pv[c.blocks[tab + j // bt], 0, j % bt] = K[j]
        c.Kb[base:base + M] = K[P:]
    return c


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
