"""Closed forms of the attention on the GPU, with no checker in between: inputs whose result the softmax
algebra fixes exactly or to a plain mean, on both kernels and every head dim.

  - a window of one position: every row sees itself only, so O is its own V row, bit for bit
    (weight exp2(0) = 1, l = 1: no rounding anywhere), also across tile, page and split boundaries;
  - an empty cache and one row: the same through the batch-key path alone;
  - q = 0: every visible key gets the same weight, so O is the mean of the visible V rows
    (float64 mean of the stored values; tolerance the path's 2e-3);
  - all keys equal: the same mean whatever q is.
"""
import numpy as np
import pytest

from espetero_amd import abi, device

from helpers import f32, small_case

pytestmark = pytest.mark.gpu

GEOM = [(8, 2, 128), (4, 2, 256), (16, 2, 512), (4, 4, 128)]


def _run(case, rows):
    from gpu_utils import run_case
    device.init(0)
    case.params.rows_per_tile = rows
    print(f"closed form: HD={case.params.head_dim} H={case.params.H} Hkv={case.params.Hkv} rows/tile={rows} seqs={case.meta['seqs']}", flush=True)
    return run_case(case)


def _own_v(case):
    """V row of every query row, repeated for the query heads of its KV head: [rows][H * HD] storage bits."""
    p = case.params
    G = p.H // p.Hkv
    v = case.Vb.reshape(case.n_rows, p.Hkv, 1, p.head_dim)
    return np.broadcast_to(v, (case.n_rows, p.Hkv, G, p.head_dim)).reshape(case.n_rows, -1)


@pytest.mark.parametrize("H,Hkv,HD", GEOM)
@pytest.mark.parametrize("seqs,rows", [(((70, 1), (0, 1), (300, 1)), 1), (((45, 150), (0, 37)), 0), (((130, 9),), 4)])
def test_window_of_one_returns_the_rows_own_v_exactly(H, Hkv, HD, seqs, rows):
    case = small_case(3, H=H, Hkv=Hkv, HD=HD, seqs=seqs, window=1)
    rows = rows or device.plan_hint3(case.params)[2]
    got = _run(case, rows)
    assert np.array_equal(got, _own_v(case))


@pytest.mark.parametrize("H,Hkv,HD", GEOM)
@pytest.mark.parametrize("dtype", [abi.ESP_F16, abi.ESP_BF16])
def test_empty_cache_single_row_returns_its_v_exactly(H, Hkv, HD, dtype):
    case = small_case(4, H=H, Hkv=Hkv, HD=HD, dtype=dtype, seqs=((0, 1), (0, 1), (0, 1)))
    got = _run(case, 1)
    assert np.array_equal(got, _own_v(case))


def _visible_mean(case):
    """Mean over each row's causally visible V rows (cached keys, then the batch rows up to itself), float64."""
    from oracle import binding as ob
    p = case.params
    G = p.H // p.Hkv
    out = np.zeros((case.n_rows, p.Hkv, p.head_dim))
    for t in case.trees:
        base, P, table, M = (int(t[k]) for k in ("base", "P", "table", "M"))
        cached = f32(ob.kv_gather(p, case.pool_ref, case.blocks[table:], P)[1], p.dtype).astype(np.float64) if P else np.zeros((0, p.kv_ld))
        batch = f32(case.Vb[base:base + M], p.dtype).astype(np.float64)
        run = cached.sum(0)
        for i in range(M):
            run = run + batch[i]
            out[base + i] = (run / (P + i + 1)).reshape(p.Hkv, p.head_dim)
    return np.broadcast_to(out[:, :, None, :], (case.n_rows, p.Hkv, G, p.head_dim)).reshape(case.n_rows, -1)


@pytest.mark.parametrize("H,Hkv,HD", GEOM)
@pytest.mark.parametrize("seqs,rows", [(((1000, 1), (33, 1), (4100, 1)), 1), (((200, 140), (0, 20)), 0), (((515, 4),), 4)])
def test_zero_query_gives_the_mean_of_the_visible_v_rows(H, Hkv, HD, seqs, rows):
    case = small_case(5, H=H, Hkv=Hkv, HD=HD, seqs=seqs)
    case.Q[:] = 0
    rows = rows or device.plan_hint3(case.params)[2]
    got = f32(_run(case, rows), case.params.dtype)
    assert np.abs(got - _visible_mean(case)).max() <= 2e-3


@pytest.mark.parametrize("H,Hkv,HD", GEOM)
def test_equal_keys_give_the_mean_whatever_the_query(H, Hkv, HD):
    case = small_case(6, H=H, Hkv=Hkv, HD=HD, seqs=((700, 1), (90, 40)))
    p = case.params
    key = case.Kb[0].copy()
    case.Kb[:] = key
    pv = case.pool_ref.reshape(case.n_blocks, 2, p.bt, p.kv_ld)
    pv[:, 0] = key                                                     # every cached K row as well
    for rows in (1, device.plan_hint3(p)[2]):
        got = f32(_run(case, rows), p.dtype)
        assert np.abs(got - _visible_mean(case)).max() <= 2e-3
