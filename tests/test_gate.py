"""The CPU checker's head-wise output gate (sp_head_gate, kernels/85_spark.metal:96-128) against
closed forms and a float64 restatement, and the checker's attention with a head-wise gate in its
epilogue against attention followed by the gate. The reference holds no vectors for this kernel:
parity with its Metal results is unpinned by reference-held data; the mathematics is pinned."""
import numpy as np
import pytest

from espetero_amd import abi, synth
from oracle import binding as ob


def _ulp(x, dtype):
    """One unit in the last place of the storage type at |x| (normal range)."""
    mant = 10 if dtype == abi.ESP_F16 else 7
    return 2.0 ** (np.floor(np.log2(np.maximum(np.abs(x), 2.0 ** -14))) - mant)


@pytest.mark.parametrize("dtype", [abi.ESP_F16, abi.ESP_BF16])
@pytest.mark.parametrize("H,HD,D", [(16, 256, 640), (5, 64, 200), (40, 128, 96)])
def test_gate_matches_float64(dtype, H, HD, D):
    p, a = synth.make_gate(H, HD, D, dtype, 7, seed=H)
    got, dots = ob.head_gate(p, a["O"], a["X"], a["Wg"], 7, want_dots=True)
    want, dots64 = ob.head_gate_f64(p, a["O"], a["X"], a["Wg"], 7)
    assert np.allclose(dots, dots64, rtol=0, atol=2e-5 * np.sqrt(D))      # fp32 accumulation of exact products
    g = ob.to_f32(got, dtype).astype(np.float64).reshape(7, H, HD)
    # one rounding of the product (half a unit) + the gate's fp32 error
    assert np.all(np.abs(g - want) <= 0.51 * _ulp(want, dtype) + 1e-6)


def test_gate_closed_forms():
    p, a = synth.make_gate(8, 128, 256, abi.ESP_F16, 5, seed=1)
    O = a["O"]
    o = ob.to_f32(O, p.dtype)
    # x == 0: every gate is sigmoid(0) = 1/2, and halving is exact in fp16 wherever the half is still normal
    X0 = np.zeros_like(a["X"])
    got = ob.to_f32(ob.head_gate(p, O, X0, a["Wg"], 5), p.dtype)
    normal = np.abs(o) >= 2.0 ** -13
    assert normal.mean() > 0.99 and np.array_equal(got[normal], (o * 0.5)[normal])
    assert np.all(np.abs(got - o * 0.5) <= 2.0 ** -25)
    # a one-hot gate row picks one input element: gate = sigmoid(c * x[row, k])
    W = np.zeros((8, 256), np.float32)
    for h in range(8):
        W[h, 17 * h + 3] = 2.0
    Wb = ob.from_f32(W, p.dtype)
    got, dots = ob.head_gate(p, O, a["X"], Wb, 5, want_dots=True)
    x = ob.to_f32(a["X"], p.dtype)
    for h in range(8):
        assert np.array_equal(dots[:, h], 2.0 * x[:, 17 * h + 3])
        g = (1.0 / (1.0 + np.exp(-dots[:, h].astype(np.float64))))[:, None]
        want = o[:, h * 128:(h + 1) * 128].astype(np.float64) * g
        assert np.all(np.abs(ob.to_f32(got[:, h * 128:(h + 1) * 128], p.dtype) - want) <= 0.51 * _ulp(want, p.dtype) + 1e-7)
    # saturated dots: +large leaves O as it is, -large clears it; head h alternates
    Xs = ob.from_f32(np.full((5, 256), 8.0, np.float32), p.dtype)
    Ws = ob.from_f32(np.where(np.arange(8)[:, None] % 2 == 0, 1.0, -1.0) * np.ones((8, 256), np.float32), p.dtype)
    got = ob.to_f32(ob.head_gate(p, O, Xs, Ws, 5), p.dtype).reshape(5, 8, 128)
    assert np.array_equal(got[:, 0::2], o.reshape(5, 8, 128)[:, 0::2])
    assert np.all(got[:, 1::2] == 0.0)


def test_gate_strides_and_untouched_padding():
    p, a = synth.make_gate(6, 64, 128, abi.ESP_F16, 4, seed=3, q_ld=6 * 64 + 24, x_ld=128 + 8)
    got = ob.head_gate(p, a["O"], a["X"], a["Wg"], 4)
    assert np.array_equal(got[:, 6 * 64:], a["O"][:, 6 * 64:])            # columns past H * head_dim
    pd, ad = synth.make_gate(6, 64, 128, abi.ESP_F16, 4, seed=3)
    dense = ob.head_gate(pd, np.ascontiguousarray(a["O"][:, :6 * 64]), np.ascontiguousarray(a["X"][:, :128]), a["Wg"], 4)
    assert np.array_equal(got[:, :6 * 64], dense)


@pytest.mark.parametrize("dtype", [abi.ESP_F16, abi.ESP_BF16])
def test_attention_with_headwise_gate_equals_attention_then_gate(dtype):
    """gate_headwise = 1 on the attention == the two-step form up to the second rounding the two-step form makes."""
    c = synth.make_case("g", 11, 4, 2, 128, dtype, 16, [(40, 3), (17, 1)], rows_per_tile=8)
    pg, ag = synth.make_gate(4, 128, 64, dtype, c.n_rows, seed=12)
    dots = ob.head_gate(pg, None, ag["X"], ag["Wg"], c.n_rows, want_dots=True)[1]
    plain = ob.attn_direct(c.params, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees)
    two_step = ob.head_gate(pg, plain, ag["X"], ag["Wg"], c.n_rows)
    p = c.params
    keep = np.ascontiguousarray(dots)
    p.gate, p.gate_ld, p.gate_hs, p.gate_off, p.gate_headwise = keep.ctypes.data, 4, 1, 0, 1
    fused = ob.attn_direct(p, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees)
    p.gate, p.gate_headwise = None, 0
    f, t = ob.to_f32(fused, dtype).astype(np.float64), ob.to_f32(two_step, dtype).astype(np.float64)
    assert np.all(np.abs(f - t) <= 1.01 * _ulp(t, dtype) + 1e-7)
    assert not np.array_equal(fused, plain)
    # and against float64: the brute force with one gate per (row, head)
    want = ob.brute_force(p, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees, gate=dots[:, :, None])
    tol = 2e-3 if dtype == abi.ESP_F16 else 1.6e-2
    assert np.abs(f.reshape(want.shape) - want).max() < tol
