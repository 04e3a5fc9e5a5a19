"""esp_head_gate on the GPU against the CPU checker, through the C ABI, and the attention kernels'
head-wise gate epilogue against attention followed by the gate. Bar: the fp32 dots within the
rounding of a differently ordered fp32 sum; gated outputs within one unit in the last place of the
storage type (the gate's last fp32 bits can move the one rounding), which at the |O| < 2 of these
inputs is below the 2e-3 the path's contract states for fp16."""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, synth
from oracle import binding as ob

from helpers import f32, small_case

pytestmark = pytest.mark.gpu


def _dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _ulps(got_bits, want_bits):
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    return np.abs(key(got_bits) - key(want_bits))


@pytest.mark.parametrize("H,HD,D,n_rows", [(16, 256, 2560, 37), (5, 64, 200, 3), (40, 128, 1024, 16), (64, 128, 4096, 50),
                                           (33, 24, 72, 17), (8, 1024, 256, 2)])
@pytest.mark.parametrize("dtype", [abi.ESP_F16, abi.ESP_BF16])
def test_gate_matches_checker(H, HD, D, n_rows, dtype):
    device.init(0)
    print(f"gate H={H} HD={HD} D={D} rows={n_rows} dtype={dtype}", flush=True)
    p, a = synth.make_gate(H, HD, D, dtype, n_rows, seed=H + n_rows)
    want, want_dots = ob.head_gate(p, a["O"], a["X"], a["Wg"], n_rows, want_dots=True)
    O = _dev(a["O"].view(np.int16))
    dots = torch.full((n_rows, H), 7.0, dtype=torch.float32, device="cuda")
    device.head_gate(p, O, _dev(a["X"].view(np.int16)), _dev(a["Wg"].view(np.int16)), dots, n_rows)
    torch.cuda.synchronize()
    assert np.abs(dots.cpu().numpy() - want_dots).max() <= 2e-5 * np.sqrt(D)
    u = _ulps(_bits(O), want)
    assert u.max() <= 1, int(u.max())
    assert (u > 0).mean() < 0.01
    if dtype == abi.ESP_F16:
        assert np.abs(ob.to_f32(_bits(O), dtype) - ob.to_f32(want, dtype)).max() <= 2e-3


def test_gate_strides_padding_and_modes():
    """Row strides wider than the data; columns past H * head_dim stay as they were; O alone, dots alone."""
    device.init(0)
    p, a = synth.make_gate(6, 64, 128, abi.ESP_F16, 21, seed=3, q_ld=6 * 64 + 24, x_ld=128 + 8)
    want, want_dots = ob.head_gate(p, a["O"], a["X"], a["Wg"], 21, want_dots=True)
    X, Wg = _dev(a["X"].view(np.int16)), _dev(a["Wg"].view(np.int16))
    O = _dev(a["O"].view(np.int16))
    device.head_gate(p, O, X, Wg, None, 21)
    dots = torch.zeros((21, 6), dtype=torch.float32, device="cuda")
    O2 = _dev(a["O"].view(np.int16))
    device.head_gate(p, None, X, Wg, dots, 21)
    torch.cuda.synchronize()
    assert _ulps(_bits(O), want).max() <= 1
    assert np.array_equal(_bits(O)[:, 6 * 64:], a["O"][:, 6 * 64:])
    assert np.array_equal(_bits(O2), a["O"])                              # the dots-only call leaves O alone
    assert np.abs(dots.cpu().numpy() - want_dots).max() <= 1e-4
    with pytest.raises(abi.EspError):
        device.head_gate(p, None, X, Wg, None, 21)
    p.D = 100
    with pytest.raises(abi.EspError):
        device.head_gate(p, O, X, Wg, None, 21)


@pytest.mark.parametrize("kw", [
    dict(seqs=((200, 1), (50, 1)), rows_per_tile=1),                                    # streaming kernel, unsplit
    dict(seqs=((5000, 1), (17, 1)), rows_per_tile=1),                                   # split: the gate sits in the merge
    dict(seqs=((300, 130), (17, 5)), rows_per_tile=128, H=4, Hkv=2),                    # tiled kernel
    dict(seqs=((64, 256),), rows_per_tile=128, H=10, Hkv=2, dtype=abi.ESP_BF16),        # tiled, bf16, GQA 5
])
def test_attention_headwise_gate_is_attention_then_gate(kw):
    """params.gate_headwise = 1 with the dots of esp_head_gate == attention, then esp_head_gate in place, up to
    the second rounding of the two-step form (one unit in the last place); and == the checker's two-step form."""
    from gpu_utils import run_case
    device.init(0)
    c = small_case(seed=51, **kw)
    p = c.params
    print(f"headwise gate {kw}", flush=True)
    pg, ag = synth.make_gate(p.H, p.head_dim, 192, p.dtype, c.n_rows, seed=52, q_ld=p.q_ld)
    X, Wg = _dev(ag["X"].view(np.int16)), _dev(ag["Wg"].view(np.int16))
    dots = torch.zeros((c.n_rows, p.H), dtype=torch.float32, device="cuda")
    device.head_gate(pg, None, X, Wg, dots, c.n_rows)
    plain = run_case(c)
    two_step = _dev(np.ascontiguousarray(plain).view(np.int16))
    device.head_gate(pg, two_step, X, Wg, None, c.n_rows)
    p.gate, p.gate_ld, p.gate_hs, p.gate_off, p.gate_headwise = dots.data_ptr(), p.H, 1, 0, 1
    fused = run_case(c)
    p.gate, p.gate_headwise = None, 0
    torch.cuda.synchronize()
    u = _ulps(np.ascontiguousarray(fused).view(np.uint16), _bits(two_step))
    assert u.max() <= 2 and (u > 1).mean() < 1e-3, int(u.max())          # 2: only just below a power of two
    want = ob.head_gate(pg, ob.attn_direct(p, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees, n_threads=8),
                        ag["X"], ag["Wg"], c.n_rows)
    tol = 2e-3 if p.dtype == abi.ESP_F16 else 8e-3
    assert np.abs(f32(fused, p.dtype) - ob.to_f32(want, p.dtype)).max() <= tol
