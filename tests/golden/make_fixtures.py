"""Writes the golden fixtures of this directory: small seeded inputs (storage bits, records) with expected
outputs computed in float64 by formulas that share no code with the C checker or the HIP kernels:

  attention_<name>.npz  inputs of one esp_attn_forward call + O from the dense float64 brute force
                        (explicit visibility matrix, one softmax per row, no paging, no online softmax)
  prep_<kind>.npz       inputs of one esp_attn_prep call + Q / K / V from the float64 closed forms
  gate.npz              inputs of one esp_head_gate call + gated O and dots in float64
  planner.json          the reference planning rule (src/model/impl/forest.h:1378-1433, gemma.h:77-116)
                        evaluated by the Python restatement on the benchmark shapes: tile, merge-job and
                        part counts and the first and last tile records

The reference's own tests hold no vectors for this path (its parity tests compare against a dylib that
is not in its tree), so these fixtures are generated here. Run from the repository root:
    python tests/golden/make_fixtures.py
The files are loaded with numpy.load(allow_pickle=False) / json.
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from espetero_amd import abi, synth  # noqa: E402
from oracle import binding as ob  # noqa: E402
from oracle import host_oracle as ho  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

ATTENTION = {
    # name: (seed, H, Hkv, HD, dtype, bt, seqs, kwargs)
    "decode_gqa8": (101, 8, 1, 128, abi.ESP_F16, 16, [(70, 1), (33, 1), (1, 1)], dict(rows_per_tile=1)),
    "decode_bf16_g5": (102, 5, 1, 128, abi.ESP_BF16, 16, [(95, 1)], dict(rows_per_tile=1)),
    "decode_hd256_bt64": (103, 2, 1, 256, abi.ESP_F16, 64, [(130, 1)], dict(rows_per_tile=1)),
    "verify_tree": (104, 4, 1, 128, abi.ESP_F16, 16, [(50, 4), (17, 4)], dict(rows_per_tile=4, desc_fn=lambda M: synth.verify_desc(M, 1))),
    "prefill_cached": (105, 2, 1, 128, abi.ESP_F16, 16, [(40, 24), (0, 9)], dict(rows_per_tile=8)),
    "prefill_bf16": (106, 2, 1, 128, abi.ESP_BF16, 16, [(33, 20)], dict(rows_per_tile=8)),
    "window_lists": (107, 2, 1, 128, abi.ESP_F16, 16, [(90, 6), (20, 1)], dict(rows_per_tile=8, window=32)),
    "window_rings": (108, 2, 1, 128, abi.ESP_F16, 16, [(100, 1), (45, 1)], dict(rows_per_tile=1, window=48, ring_layer=True)),
    "bidi_span": (109, 2, 1, 128, abi.ESP_F16, 16, [(20, 12)], dict(rows_per_tile=8, bidi=1, desc_fn=lambda M: synth.image_desc(M, 3, 9))),
    "wide_tree": (110, 2, 1, 128, abi.ESP_F16, 16, [(30, 10)], dict(rows_per_tile=8, desc_fn=lambda M: synth.verify_desc(M, 6))),
    "decode_hd512_g8": (111, 8, 1, 512, abi.ESP_F16, 16, [(75, 1), (20, 1)], dict(rows_per_tile=1)),
    "prefill_hd512": (112, 2, 1, 512, abi.ESP_BF16, 16, [(37, 21)], dict(rows_per_tile=64)),
}


def attention_fixtures():
    for name, (seed, H, Hkv, HD, dtype, bt, seqs, kw) in ATTENTION.items():
        c = synth.make_case(name, seed, H, Hkv, HD, dtype, bt, seqs, **kw)
        p = c.params
        O = ob.brute_force(p, c.Q, c.Kb, c.Vb, c.pool_ref, c.blocks, c.desc, c.pos, c.trees)
        meta = dict(H=H, Hkv=Hkv, head_dim=HD, dtype=int(dtype), bt=bt, window=int(p.window), ring=int(p.ring), bidi=int(p.bidi),
                    rows_per_tile=int(p.rows_per_tile), scale=float(p.scale), n_blocks=int(c.n_blocks), n_rows=int(c.n_rows))
        np.savez_compressed(os.path.join(HERE, f"attention_{name}.npz"), meta=json.dumps(meta), Q=c.Q, Kb=c.Kb, Vb=c.Vb,
                            pool_ref=c.pool_ref, blocks=c.blocks, trees=c.trees.view(np.int32).reshape(-1, 4), desc=c.desc,
                            pos=c.pos, O=O.reshape(c.n_rows, -1))


def prep_fixtures():
    for kind, H, Hkv, HD, dtype in (("qwen35", 3, 1, 256, abi.ESP_F16), ("gemma", 2, 1, 128, abi.ESP_BF16), ("omni", 5, 1, 128, abi.ESP_F16),
                                    ("gemma512", 4, 1, 512, abi.ESP_F16)):
        n = 7
        p, a = synth.make_prep("gemma" if kind == "gemma512" else kind, H, Hkv, HD, dtype, n, seed=120 + H)
        Q, K, V = ob.attn_prep_f64(p, a["X"], a["qn_w"], a["kn_w"], a["pos"], a["inv_freq"], a["rope_sel"], n)
        meta = {f[0]: getattr(p, f[0]) for f in abi.PrepParams._fields_}
        sel = np.zeros(0, np.int32) if a["rope_sel"] is None else a["rope_sel"]
        np.savez_compressed(os.path.join(HERE, f"prep_{kind}.npz"), meta=json.dumps(meta), X=a["X"], qn_w=a["qn_w"], kn_w=a["kn_w"],
                            pos=a["pos"], inv_freq=a["inv_freq"], rope_sel=sel, Q=Q, K=K, V=V)


def gate_fixture():
    n = 6
    p, a = synth.make_gate(5, 64, 200, abi.ESP_F16, n, seed=130)
    O, dots = ob.head_gate_f64(p, a["O"], a["X"], a["Wg"], n)
    meta = {f[0]: getattr(p, f[0]) for f in abi.GateParams._fields_}
    np.savez_compressed(os.path.join(HERE, "gate.npz"), meta=json.dumps(meta), O_in=a["O"], X=a["X"], Wg=a["Wg"],
                        O=O.reshape(n, -1), dots=dots)


def planner_fixture():
    lens = synth.c2_lengths()
    shapes = {
        "c1": ([(0, 1024, 0, 1)], 4),
        "c2": ([(i, L, 512 * i, 1) for i, L in enumerate(lens)], 4),
        "c3_p6144": ([(0, 6144, 0, 2048)], 8),
        "c4_decode_global": ([(i, 16384, 1024 * i, 1) for i in range(8)], 8),
        "c5": ([(4 * i, 32768, 2048 * i, 4) for i in range(8)], 4),
    }
    out = {}
    for name, (trees, groups) in shapes.items():
        tiles, jobs, parts, rows = ho.g4_plan_tiles(trees, groups, 512, 0, None)
        out[name] = dict(trees=trees, groups=groups, n_tiles=len(tiles), n_jobs=len(jobs), n_parts=parts, rows_per_tile=rows,
                         first_tile=list(tiles[0]), last_tile=list(tiles[-1]), first_job=list(jobs[0]) if jobs else None,
                         tile_sum=[int(sum(t[i] for t in tiles)) for i in range(8)])
    with open(os.path.join(HERE, "planner.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)


if __name__ == "__main__":
    attention_fixtures()
    prep_fixtures()
    gate_fixture()
    planner_fixture()
    total = sum(os.path.getsize(os.path.join(HERE, f)) for f in os.listdir(HERE) if f.endswith((".npz", ".json")))
    print(f"wrote fixtures: {total / 1024:.0f} KiB")
