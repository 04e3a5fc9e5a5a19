"""Seeded random valid shapes through the C ABI against the CPU checker: head dim, grouping, element
type, page size, decode / verify / chunk / prefill / image passes, windows over lists and rings, split
targets, head-wise gates. Each case is small enough for the checker; together they reach corners the
hand-written cases do not (two defects were found this way: a partial 16-key unit at head dim 256, a
one-row remainder tile on a sliding layer). Bar: 2e-3 beyond the stored output's own rounding (helpers.max_abs)."""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, host, synth

from helpers import max_abs, oracle_direct, small_case, tol_for

pytestmark = pytest.mark.gpu


def _draw(rng):
    HD = int(rng.choice([128, 256, 512]))
    Hkv = int(rng.choice([1, 2, 3]))
    G = int(rng.choice([1, 2, 3, 4, 6, 8, 16]))
    kind = str(rng.choice(["decode", "verify", "prefill", "smallchunk", "longdecode", "image"]))
    nseq = int(rng.integers(1, 5))
    window = int(rng.choice([0, 0, 17, 100, 1000]))
    ring = bool(window and rng.integers(0, 2))
    kw = dict(H=Hkv * G, Hkv=Hkv, HD=HD, dtype=int(rng.choice([abi.ESP_F16, abi.ESP_BF16])), bt=int(rng.choice([16, 32, 48, 64, 128])),
              window=window, ring_layer=ring, fill_unused=not ring)
    if kind == "decode":
        seqs, R = [(int(rng.integers(0, 300)), 1) for _ in range(nseq)], 1
    elif kind == "longdecode":
        seqs, R = [(int(rng.integers(1000, 7000)), 1) for _ in range(min(nseq, 2))], 1
    elif kind == "verify":
        M = int(rng.integers(2, 10))
        seqs = [(int(rng.integers(1, 2000)), M) for _ in range(nseq)]
        R, root = int(rng.choice([M, 1, 2, 4, 8])), int(rng.integers(1, M))
        kw["desc_fn"] = lambda m, root=root: synth.verify_desc(m, root)
    elif kind == "prefill":
        seqs = [(int(rng.integers(0, 1500)), int(rng.integers(1, 400))) for _ in range(min(nseq, 2))]
        R = 64 if HD == 512 else int(rng.choice([32, 64, 128]))
    elif kind == "image":
        M = int(rng.integers(4, 150))
        a0 = int(rng.integers(0, M - 2))
        b0 = int(rng.integers(a0 + 1, M + 1))
        seqs = [(int(rng.integers(0, 500)), M)]
        R = int(rng.choice([8, 64])) if HD == 512 else int(rng.choice([8, 128]))
        kw["bidi"] = 1
        kw["desc_fn"] = lambda m, a0=a0, b0=b0: synth.image_desc(m, a0, b0)
    else:
        seqs, R = [(int(rng.integers(0, 600)), int(rng.integers(1, 33))) for _ in range(nseq)], int(rng.choice([4, 8, 16]))
    if ring:
        seqs = [(max(P, 1), M) for P, M in seqs]
    split = int(rng.choice([0, 3, 8, 64, 700, 5000]))
    gate = bool(rng.integers(0, 4) == 0)
    # drawn last, so that the shapes above are those of earlier versions of this sweep: on windowed layers, now and then,
    # positions that do not rise by one per row (two rows per position, as siblings of a tree have)
    kw["paired_positions"] = bool(window and kind in ("prefill", "smallchunk", "verify") and rng.integers(0, 3) == 0)
    return kind, tuple(seqs), R, split, gate, kw


@pytest.mark.parametrize("chunk", range(6))
def test_random_shapes_match_the_checker(chunk):
    from gpu_utils import run_case
    device.init(0)
    for it in range(25 * chunk, 25 * (chunk + 1)):
        rng = np.random.default_rng(770003 + it)
        kind, seqs, R, split, gate, kw = _draw(rng)
        print(f"it={it} kind={kind} seqs={seqs} R={R} split={split} gate={gate} "
              f"{ {k: v for k, v in kw.items() if k != 'desc_fn'} }", flush=True)
        paired = kw.pop("paired_positions")
        c = small_case(seed=9000 + it, seqs=seqs, rows_per_tile=R, **kw)
        if paired:
            for t in c.trees:
                P, M, base = int(t["P"]), int(t["M"]), int(t["base"])
                c.pos[base:base + M, 0:3] = (P + np.arange(M) // 2)[:, None]
        p = c.params
        keep = None
        if gate:
            keep = np.ascontiguousarray(np.random.default_rng(it).standard_normal((c.n_rows, p.H)).astype(np.float32))
            gd = torch.from_numpy(keep).cuda()
            p.gate, p.gate_ld, p.gate_hs, p.gate_off, p.gate_headwise = gd.data_ptr(), p.H, 1, 0, 1
        got = run_case(c, host.options_mi355x(R, split) if split else None)
        if gate:
            p.gate = keep.ctypes.data      # the checker reads the same values from host memory
        want = oracle_direct(c, threads=8)
        p.gate, p.gate_headwise = None, 0
        err = max_abs(got, want, p.dtype)
        assert err <= tol_for(p.dtype), (it, kind, seqs, R, split, gate, err)
