"""Shared by the tests: small case builders and comparisons."""
import numpy as np

from espetero_amd import abi, synth
from oracle import binding as ob

TOL = 2e-3  # max-abs contract of the path (fp32 accumulation, fp16 / bf16 storage)


def f32(bits, dtype):
    return ob.to_f32(bits, dtype)


def max_abs(a_bits, b, dtype):
    """a: storage bits; b: storage bits or float array."""
    a = f32(a_bits, dtype).astype(np.float64)
    bb = f32(b, dtype).astype(np.float64) if b.dtype == np.uint16 else b.astype(np.float64).reshape(a.shape)
    return float(np.abs(a - bb).max())


def tol_for(dtype):
    # bf16 output rounding alone is 2^-9 relative; outputs here are |o| < 1.
    return TOL if dtype == abi.ESP_F16 else 4e-3


def small_case(seed=0, H=8, Hkv=2, HD=128, dtype=abi.ESP_F16, bt=16, seqs=((70, 1), (33, 1)), **kw):
    return synth.make_case("small", seed, H, Hkv, HD, dtype, bt, list(seqs), **kw)


def oracle_direct(case, threads=4):
    c = case
    return ob.attn_direct(c.params, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees, n_threads=threads)


def brute(case):
    c = case
    H, HD = c.params.H, c.params.head_dim
    return ob.brute_force(c.params, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees).reshape(c.n_rows, H * HD)
