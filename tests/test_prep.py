"""The CPU checker's attn_prep against the closed forms (RMSNorm, rotation matrix) in float64,
in the three arrangements the reference has (kernels/40_attention.metal:9-102,
80_gemma.metal:52-108, 82_qwen3_omni.metal:30-88). The reference holds no vectors for these
kernels: parity with its Metal results is unpinned by reference-held data; what is pinned is the
mathematics and the folded append."""
import numpy as np
import pytest

from espetero_amd import abi, synth
from oracle import binding as ob

KINDS = [("qwen35", 256), ("gemma", 256), ("gemma", 128), ("omni", 128), ("gemma", 512)]


def _run(kind, HD, dtype, n_rows=9, seed=5, **kw):
    p, a = synth.make_prep(kind, 6, 2, HD, dtype, n_rows, seed=seed, **kw)
    out = ob.attn_prep(p, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], n_rows)
    return p, a, out


@pytest.mark.parametrize("kind,HD", KINDS)
@pytest.mark.parametrize("dtype", [abi.ESP_F16, abi.ESP_BF16])
def test_prep_matches_float64_closed_forms(kind, HD, dtype):
    p, a, out = _run(kind, HD, dtype)
    want = ob.attn_prep_f64(p, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], 9)
    ulp = 2.0 ** -11 if dtype == abi.ESP_F16 else 2.0 ** -8      # half a unit in the last place, relative
    for got, w in zip(out, want):
        g = ob.to_f32(got, dtype).astype(np.float64)
        assert np.all(np.abs(g - w) <= 1.02 * ulp * np.abs(w) + 1e-6)


def test_rotation_preserves_pair_norms_and_position_zero_is_identity():
    p, a = synth.make_prep("omni", 4, 2, 128, abi.ESP_F16, 6, seed=2)
    q, k, _ = ob.attn_prep_f64(p, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], 6)
    pos0 = np.zeros_like(a["pos"])
    q0, k0, _ = ob.attn_prep_f64(p, a["X"], a["qn_w"], a["kn_w"], pos0, a["inv_freq"], a["rope_sel"], 6)
    for y, y0 in ((q, q0), (k, k0)):
        y, y0 = y.reshape(6, -1, 128), y0.reshape(6, -1, 128)
        assert np.allclose(y[..., :64] ** 2 + y[..., 64:] ** 2, y0[..., :64] ** 2 + y0[..., 64:] ** 2, rtol=1e-12)
    # position 0: the checker's output is the normalised, weighted, scaled input itself
    Q, K, V = ob.attn_prep(p, a["X"], a["qn_w"], a["kn_w"], pos0, a["inv_freq"], a["rope_sel"], 6)
    x = a["X"].astype(np.float64)[:, :128]
    want = x / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6) * a["qn_w"] * p.q_scale
    assert np.allclose(ob.to_f32(Q[:, :128], p.dtype), want, rtol=2.0 ** -10, atol=1e-6)
    assert np.array_equal(V, ob.from_f32(a["X"][:, p.v_off:], p.dtype))            # values: the cast alone


def test_partial_rotation_leaves_the_other_dims_alone():
    """qwen35 arrangement: 64 of 256 dims rotate (40_:58-71); the gate columns beside q are not read."""
    p, a = synth.make_prep("qwen35", 4, 2, 256, abi.ESP_F16, 4, seed=3)
    Q, K, _ = ob.attn_prep(p, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], 4)
    Q0, K0, _ = ob.attn_prep(p, a["X"], a["qn_w"], a["kn_w"], np.zeros_like(a["pos"]), a["inv_freq"], a["rope_sel"], 4)
    assert np.array_equal(Q.reshape(4, 4, 256)[..., 64:], Q0.reshape(4, 4, 256)[..., 64:])
    assert not np.array_equal(Q.reshape(4, 4, 256)[..., :64], Q0.reshape(4, 4, 256)[..., :64])
    X2 = a["X"].copy()
    for h in range(4):
        X2[:, h * 512 + 256:(h + 1) * 512] = 777.0                                # the gates
    Q2, _, _ = ob.attn_prep(p, X2, a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], 4)
    assert np.array_equal(Q, Q2)


def test_component_selection_per_frequency():
    """Frequency f rotates by position component rope_sel[f] (40_:62-63, 82_:77-79)."""
    p, a = synth.make_prep("omni", 2, 1, 128, abi.ESP_F16, 3, seed=4)
    base = ob.attn_prep(p, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], 3)[0].reshape(3, 2, 128)
    pos2 = a["pos"].copy()
    pos2[:, 1] += 5                                                                # the height component only
    moved = ob.attn_prep(p, a["X"], a["qn_w"], a["kn_w"], pos2, a["inv_freq"], a["rope_sel"], 3)[0].reshape(3, 2, 128)
    f = np.arange(64)
    touched = np.concatenate([f[a["rope_sel"] == 1], f[a["rope_sel"] == 1] + 64])
    same = np.setdiff1d(np.arange(128), touched)
    assert np.array_equal(base[..., same], moved[..., same])
    assert not np.array_equal(base[..., touched], moved[..., touched])


def test_folded_append_equals_kv_save_of_the_outputs():
    """40_:86-100: the prep kernel writes the row's K / V into its pool entries; the pool must end up
    as a kv_save (40_:875-889) of the same rows would leave it, including a row saved into two slots."""
    n_rows, bt, n_blocks = 7, 16, 6
    p, a = synth.make_prep("qwen35", 4, 2, 256, abi.ESP_F16, n_rows, seed=6, bt=bt)
    table = np.full((n_rows, 4), -1, np.int32)
    entries = []
    for r in range(n_rows):
        table[r, :2] = (r % n_blocks, (3 * r) % bt)
        entries.append((r, r % n_blocks, (3 * r) % bt, 0))
    table[2, 2:] = (5, 9)                                                          # row 2 goes to a second slot too
    entries.append((2, 5, 9, 0))
    pool = np.zeros(n_blocks * 2 * bt * p.kv_ld, np.uint16)
    _, Kb, Vb = ob.attn_prep(p, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], n_rows, table, pool)
    ap = synth.make_params(4, 2, 256, abi.ESP_F16, bt)
    want = np.zeros_like(pool)
    ob.kv_save(ap, Kb, Vb, want, np.array(entries, abi.KVSAVE_DT))
    assert np.array_equal(pool, want) and pool.any()
