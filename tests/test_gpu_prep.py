"""esp_attn_prep on the GPU against the CPU checker, through the C ABI. Bar: every output within one
unit in the last place of the storage type of the checker's (rsqrt / sin / cos differ in their last
fp32 bits between the two, which can move a rounding), or, where a rotation cancels to a small value,
within half a unit in the last place at 1.0 in absolute terms; the folded append bit-identical to
esp_kv_save of the kernel's own outputs."""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, synth
from oracle import binding as ob

pytestmark = pytest.mark.gpu


def _dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _ulps(got_bits, want_bits, dtype):
    """Distance in units of the last place between two arrays of storage bits (sign-magnitude order)."""
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    return np.abs(key(got_bits) - key(want_bits))


def _run_gpu(p, a, n_rows, table=None, pool=None):
    tdt = torch.float16 if p.dtype == abi.ESP_F16 else torch.bfloat16
    Q = torch.zeros(n_rows, p.q_ld, dtype=tdt, device="cuda")
    Kb = torch.zeros(n_rows, p.kv_ld, dtype=tdt, device="cuda")
    Vb = torch.zeros_like(Kb)
    device.attn_prep(p, _dev(a["X"]), _dev(a["qn_w"]), _dev(a["kn_w"]), _dev(a["pos"]), _dev(a["inv_freq"]), _dev(a["rope_sel"]),
                     Q, Kb, Vb, _dev(table), pool, n_rows)
    torch.cuda.synchronize()
    bits = lambda t: t.view(torch.int16).cpu().numpy().view(np.uint16)  # noqa: E731
    return bits(Q), bits(Kb), bits(Vb)


@pytest.mark.parametrize("kind,H,Hkv,HD", [("qwen35", 8, 2, 256), ("gemma", 16, 8, 256), ("gemma", 8, 2, 128),
                                            ("omni", 40, 8, 128), ("omni", 3, 1, 128),
                                            ("gemma", 16, 2, 512), ("omni", 5, 1, 512)])  # 512: g4_attn_prep512, 80_gemma.metal:113
@pytest.mark.parametrize("dtype", [abi.ESP_F16, abi.ESP_BF16])
def test_prep_matches_checker(kind, H, Hkv, HD, dtype):
    device.init(0)
    n_rows = 37
    p, a = synth.make_prep(kind, H, Hkv, HD, dtype, n_rows, seed=8)
    print(f"prep {kind} H={H} Hkv={Hkv} HD={HD} dtype={dtype}", flush=True)
    want = ob.attn_prep(p, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], n_rows)
    got = _run_gpu(p, a, n_rows)
    half_ulp_at_1 = 2.0 ** -11 if dtype == abi.ESP_F16 else 2.0 ** -8
    for g, w, name in zip(got, want, "QKV"):
        u = _ulps(g, w, dtype)
        # One unit in the last place; where a rotation cancels (x cos - partner sin near 0) the result is small
        # and its last place is finer than the error of its two terms: there the absolute difference counts.
        far = (u > 1) & (np.abs(ob.to_f32(g, dtype) - ob.to_f32(w, dtype)) > half_ulp_at_1)
        assert not far.any(), (name, int(u.max()))
        assert (u > 0).mean() < 0.02, (name, float((u > 0).mean()))       # and almost all bit-identical
    assert np.array_equal(got[2], want[2]) or p.v_norm                    # a plain cast has nothing to differ in


def test_prep_folded_append_is_bitwise_kv_save():
    device.init(0)
    n_rows, bt, n_blocks = 50, 16, 12
    p, a = synth.make_prep("omni", 10, 2, 128, abi.ESP_BF16, n_rows, seed=9, bt=bt)
    rng = np.random.default_rng(9)
    slots = rng.permutation(n_blocks * bt)[:n_rows + 1]                    # distinct (block, position) targets
    table = np.full((n_rows, 4), -1, np.int32)
    entries = []
    for r in range(n_rows):
        if r % 7 == 3:
            continue                                                       # a row that is not saved
        table[r, :2] = (slots[r] // bt, slots[r] % bt)
        entries.append((r, slots[r] // bt, slots[r] % bt, 0))
    table[5, 2:] = (slots[n_rows] // bt, slots[n_rows] % bt)               # one row into two slots
    entries.append((5, slots[n_rows] // bt, slots[n_rows] % bt, 0))
    ap = synth.make_params(10, 2, 128, abi.ESP_BF16, bt)
    pool = torch.zeros(n_blocks * 2 * bt * p.kv_ld, dtype=torch.bfloat16, device="cuda")
    _, Kb, Vb = _run_gpu(p, a, n_rows, table, pool)
    want = torch.zeros_like(pool)
    e = np.array(entries, abi.KVSAVE_DT)
    device.kv_save(ap, _dev(Kb.view(np.int16)), _dev(Vb.view(np.int16)), want, device.to_dev(e), len(e))
    torch.cuda.synchronize()
    assert torch.equal(pool.view(torch.int16), want.view(torch.int16)) and bool(pool.any())


@pytest.mark.parametrize("kind,H,Hkv,HD,dtype,first", [("omni", 10, 2, 128, abi.ESP_BF16, 0), ("qwen35", 4, 2, 256, abi.ESP_F16, 0),
                                                       ("gemma", 4, 4, 256, abi.ESP_F16, 8), ("omni", 6, 2, 128, abi.ESP_F16, 5),
                                                       ("gemma", 8, 2, 512, abi.ESP_F16, 0), ("gemma", 4, 1, 512, abi.ESP_BF16, 3)])
def test_prep_folded_append_of_a_prefill_chunk(kind, H, Hkv, HD, dtype, first):
    """Rows at consecutive positions of scattered pages, as a prefill chunk appends them: groups of 8 rows
    at 8-aligned positions leave as 16-byte stores of the transposed V plane, the ragged last group and
    a chunk that starts off the 8-token grid (first = 5) as element stores. Same bits either way."""
    device.init(0)
    n_rows, bt = 77, 16
    n_blocks = (first + n_rows + bt - 1) // bt + 2
    p, a = synth.make_prep(kind, H, Hkv, HD, dtype, n_rows, seed=10, bt=bt)
    pages = np.random.default_rng(10).permutation(n_blocks).astype(np.int32)
    token = first + np.arange(n_rows)
    table = np.full((n_rows, 4), -1, np.int32)
    table[:, 0], table[:, 1] = pages[token // bt], token % bt
    e = np.zeros(n_rows, abi.KVSAVE_DT)
    e["src_row"], e["block"], e["pos"] = np.arange(n_rows), table[:, 0], table[:, 1]
    tdt = torch.float16 if dtype == abi.ESP_F16 else torch.bfloat16
    pool = torch.zeros(n_blocks * 2 * bt * p.kv_ld, dtype=tdt, device="cuda")
    _, Kb, Vb = _run_gpu(p, a, n_rows, table, pool)
    ap = synth.make_params(H, Hkv, HD, dtype, bt)
    want = torch.zeros_like(pool)
    device.kv_save(ap, _dev(Kb.view(np.int16)), _dev(Vb.view(np.int16)), want, device.to_dev(e), n_rows)
    torch.cuda.synchronize()
    assert torch.equal(pool.view(torch.int16), want.view(torch.int16)) and bool(pool.any())


def test_prep_rejects_bad_arguments():
    device.init(0)
    p, a = synth.make_prep("omni", 4, 2, 128, abi.ESP_F16, 4)
    p.rope_dims = 48
    with pytest.raises(abi.EspError):
        _run_gpu(p, a, 4)
    p.rope_dims = 128
    p.head_dim = 64
    with pytest.raises(abi.EspError):
        _run_gpu(p, a, 4)
