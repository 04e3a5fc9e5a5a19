"""Seeded random shapes for the entry points either side of the attention - esp_attn_prep (with and without the
folded append), esp_head_gate, the pool maintenance calls - through the C ABI against the CPU checker. Bars as in
the hand-written tests: prep within one unit in the last place (absolute half a unit at 1.0 where a rotation
cancels), append and pool contents bit-exact, gate within one unit in the last place."""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, synth
from oracle import binding as ob

pytestmark = pytest.mark.gpu


def _dev(x):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _ulps(g, w):
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    return np.abs(key(g) - key(w))


@pytest.mark.parametrize("chunk", range(3))
def test_random_prep_calls(chunk):
    device.init(0)
    for it in range(12 * chunk, 12 * (chunk + 1)):
        rng = np.random.default_rng(41000 + it)
        dtype = int(rng.choice([abi.ESP_F16, abi.ESP_BF16]))
        tdt = torch.float16 if dtype == abi.ESP_F16 else torch.bfloat16
        kind = str(rng.choice(["qwen35", "gemma", "omni"]))
        HD, Hkv = int(rng.choice([128, 256, 512])), int(rng.choice([1, 2, 3, 8]))
        H = Hkv * int(rng.choice([1, 2, 5, 8]))
        n_rows, bt = int(rng.integers(1, 90)), int(rng.choice([16, 32, 64]))
        p, a = synth.make_prep(kind, H, Hkv, HD, dtype, n_rows, seed=it, bt=bt)
        if rng.integers(0, 2):   # a narrower rotation than the arrangement's own
            p.rope_dims = int(rng.choice([16, 32, 64, HD]))
            half = p.rope_dims // 2
            a["inv_freq"] = (1e6 ** (-np.arange(half) / half)).astype(np.float32)
            a["rope_sel"] = None if a["rope_sel"] is None else (np.arange(half) % 3).astype(np.int32)
        mode = str(rng.choice(["none", "chunk", "scatter"]))
        n_blocks = (n_rows + 40) // bt + 3
        table = pool = None
        if mode != "none":
            table = np.full((n_rows, 4), -1, np.int32)
            if mode == "chunk":      # consecutive positions of scattered pages, from an arbitrary first token
                pages = rng.permutation(n_blocks).astype(np.int32)
                tok = int(rng.integers(0, 30)) + np.arange(n_rows)
                table[:, 0], table[:, 1] = pages[tok // bt], tok % bt
            else:                    # unrelated (block, position) targets, one row not saved
                slots = rng.permutation(n_blocks * bt)[:n_rows]
                table[:, 0], table[:, 1] = slots // bt, slots % bt
                if n_rows > 3:
                    table[2, :2] = -1
            pool = torch.zeros(n_blocks * 2 * bt * p.kv_ld, dtype=tdt, device="cuda")
        print(f"it={it} prep {kind} H={H} Hkv={Hkv} HD={HD} dt={dtype} rows={n_rows} bt={bt} rope={p.rope_dims} {mode}", flush=True)
        Q = torch.zeros(n_rows, p.q_ld, dtype=tdt, device="cuda")
        Kb = torch.zeros(n_rows, p.kv_ld, dtype=tdt, device="cuda")
        Vb = torch.zeros_like(Kb)
        device.attn_prep(p, _dev(a["X"]), _dev(a["qn_w"]), _dev(a["kn_w"]), _dev(a["pos"]), _dev(a["inv_freq"]), _dev(a["rope_sel"]),
                         Q, Kb, Vb, _dev(table), pool, n_rows)
        torch.cuda.synchronize()
        want = ob.attn_prep(p, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], n_rows)
        half_ulp = 2.0 ** -11 if dtype == abi.ESP_F16 else 2.0 ** -8
        for g, w, name in zip((_bits(Q), _bits(Kb), _bits(Vb)), want, "QKV"):
            far = (_ulps(g, w) > 1) & (np.abs(ob.to_f32(g, dtype) - ob.to_f32(w, dtype)) > half_ulp)
            assert not far.any(), (it, name)
        if pool is not None:
            ap = synth.make_params(H, Hkv, HD, dtype, bt)
            ent = np.array([(r, table[r, 0], table[r, 1], 0) for r in range(n_rows) if table[r, 0] >= 0], abi.KVSAVE_DT)
            want_pool = torch.zeros_like(pool)
            device.kv_save(ap, Kb.view(torch.int16), Vb.view(torch.int16), want_pool, device.to_dev(ent), len(ent))
            torch.cuda.synchronize()
            assert torch.equal(pool.view(torch.int16), want_pool.view(torch.int16)), it


def test_random_gate_calls():
    device.init(0)
    for it in range(30):
        rng = np.random.default_rng(42000 + it)
        dtype = int(rng.choice([abi.ESP_F16, abi.ESP_BF16]))
        H, HD = int(rng.integers(1, 65)), int(rng.choice([8, 24, 64, 128, 256, 512, 1024]))
        D, n_rows = 8 * int(rng.integers(1, 600)), int(rng.integers(1, 70))
        p, a = synth.make_gate(H, HD, D, dtype, n_rows, seed=it, q_ld=H * HD + 8 * int(rng.integers(0, 3)), x_ld=D + 8 * int(rng.integers(0, 3)))
        print(f"it={it} gate H={H} HD={HD} D={D} rows={n_rows} dt={dtype}", flush=True)
        want, want_dots = ob.head_gate(p, a["O"], a["X"], a["Wg"], n_rows, want_dots=True)
        O = _dev(a["O"].view(np.int16))
        dots = torch.zeros((n_rows, H), dtype=torch.float32, device="cuda")
        device.head_gate(p, O, _dev(a["X"].view(np.int16)), _dev(a["Wg"].view(np.int16)), dots, n_rows)
        torch.cuda.synchronize()
        assert _ulps(O.cpu().numpy().view(np.uint16), want).max() <= 1, it
        assert np.abs(dots.cpu().numpy() - want_dots).max() <= 2e-5 * np.sqrt(D) + 1e-5, it


def test_random_pool_maintenance():
    from gpu_utils import dev_u16, to_host_u16
    device.init(0)
    for it in range(30):
        rng = np.random.default_rng(43000 + it)
        dtype = int(rng.choice([abi.ESP_F16, abi.ESP_BF16]))
        HD, Hkv, bt = int(rng.choice([128, 256, 512])), int(rng.choice([1, 2, 3, 8])), int(rng.choice([16, 32, 48, 64, 128]))
        p = synth.make_params(Hkv, Hkv, HD, dtype, bt)
        n_blocks = int(rng.integers(4, 30))
        print(f"it={it} pool HD={HD} Hkv={Hkv} bt={bt} blocks={n_blocks}", flush=True)
        ref = rng.integers(0, 65536, n_blocks * 2 * bt * p.kv_ld).astype(np.uint16)
        nat = torch.zeros_like(dev_u16(ref))
        device.kv_relayout(p, dev_u16(ref), abi.ESP_LAYOUT_REFERENCE, nat, abi.ESP_LAYOUT_NATIVE, n_blocks)
        rows = min(int(rng.integers(1, 120)), n_blocks * bt)
        Kb = rng.integers(0, 65536, (rows, p.kv_ld)).astype(np.uint16)
        Vb = rng.integers(0, 65536, (rows, p.kv_ld)).astype(np.uint16)
        if rng.integers(0, 2):       # a chunk's append: consecutive tokens through a shuffled table
            table = rng.permutation(n_blocks).astype(np.int32)
            tok = int(rng.integers(0, n_blocks * bt - rows + 1)) + np.arange(rows)
            ent = np.array([(r, int(table[tok[r] // bt]), int(tok[r] % bt), 0) for r in range(rows)], abi.KVSAVE_DT)
        else:                        # decode rows of unrelated sequences
            slots = rng.permutation(n_blocks * bt)[:rows]
            ent = np.array([(r, int(slots[r] // bt), int(slots[r] % bt), 0) for r in range(rows)], abi.KVSAVE_DT)
        device.kv_save(p, dev_u16(Kb), dev_u16(Vb), nat, device.to_dev(ent), len(ent))
        ob.kv_save(p, Kb, Vb, ref, ent)
        back = torch.zeros_like(nat)
        device.kv_relayout(p, nat, abi.ESP_LAYOUT_NATIVE, back, abi.ESP_LAYOUT_REFERENCE, n_blocks)
        torch.cuda.synchronize()
        assert np.array_equal(to_host_u16(back), ref), it
        tl = rng.permutation(n_blocks).astype(np.int32)[:max(1, n_blocks // 2)]
        n_tok = int(rng.integers(1, len(tl) * bt + 1))
        Kd = torch.zeros(n_tok * p.kv_ld, dtype=torch.int16, device="cuda")
        Vd = torch.zeros_like(Kd)
        device.kv_gather(p, nat, device.to_dev(tl), n_tok, Kd, Vd)
        torch.cuda.synchronize()
        Kw, Vw = ob.kv_gather(p, ref, tl, n_tok)
        assert np.array_equal(to_host_u16(Kd).reshape(n_tok, -1), Kw) and np.array_equal(to_host_u16(Vd).reshape(n_tok, -1), Vw), it
