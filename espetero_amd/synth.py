"""Seeded synthetic attention workloads (host side, numpy): the five benchmark
shapes and scaled-down variants of them for the parity tests.

A case holds logical inputs (Q, batch K/V rows, cached K/V through a block
table into a pool in the REFERENCE block layout, tree / desc / pos records).
The device pool in the native layout is made from it with esp_kv_relayout, so
the same bits reach the checker and the HIP path.
"""
from dataclasses import dataclass, field

import numpy as np

from . import abi


def _bits(x, dtype):
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dtype == abi.ESP_BF16:
        u = x.view(np.uint32)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return x.astype(np.float16).view(np.uint16)


@dataclass
class Case:
    name: str
    params: abi.AttnParams
    Q: np.ndarray          # [n_rows][H * HD] storage bits
    Kb: np.ndarray         # [n_rows][Hkv * HD]
    Vb: np.ndarray
    pool_ref: np.ndarray   # flat uint16, reference block layout, one layer region
    n_blocks: int
    blocks: np.ndarray     # int32 block table
    trees: np.ndarray      # TREE_DT
    desc: np.ndarray       # [n_rows][4] int32
    pos: np.ndarray        # [n_rows][4] int32
    n_rows: int
    meta: dict = field(default_factory=dict)


def make_params(H, Hkv, HD, dtype, bt, window=0, ring=0, scale=None, rows_per_tile=8, bidi=0):
    p = abi.AttnParams()
    p.H, p.Hkv, p.head_dim, p.dtype = H, Hkv, HD, dtype
    p.q_ld, p.kv_ld, p.bt = H * HD, Hkv * HD, bt
    p.window, p.ring, p.bidi = window, ring, bidi
    p.rows_per_tile = rows_per_tile
    p.scale = float(scale if scale is not None else HD ** -0.5)
    p.kv_base = 0
    p.gate = None
    return p


def image_desc(M, a, b):
    """Plain causal rows with one bidirectional span [a, b) (image tokens on a layer with bidi set):
    rows inside the span also see the span's later rows (80_gemma.metal:284, img_end)."""
    d = np.zeros((M, 4), np.int32)
    d[a:b, 3] = b
    return d


def verify_desc(M, root=1):
    """Rows of one verify tree: `root` pending tokens, then one hosted draft chain
    (src/model/impl/forest.h:2400-2404, 2439-2442): chain rows see the whole root and
    their own segment up to themselves."""
    d = np.zeros((M, 4), np.int32)
    d[root:, 0] = root
    d[root:, 2] = root
    return d


def make_case(name, seed, H, Hkv, HD, dtype, bt, seqs, n_blocks=None, window=0, ring_layer=False, scale=None,
              rows_per_tile=8, desc_fn=None, fill_unused=False, sigma=0.5, bidi=0):
    """seqs: list of (P cached keys, M rows this pass). Block tables: slices of one
    seeded permutation of the pool's pages (tools/qsa_check.mm:120-123 shuffles its table
    for the same reason: contiguous pages would hide addressing mistakes)."""
    rng = np.random.default_rng(seed)
    kvw = Hkv * HD
    need = sum((P + bt - 1) // bt for P, _ in seqs)
    ring = 0
    if ring_layer:
        ring = (window + bt - 1) // bt
        n_blocks = len(seqs) * ring
    elif n_blocks is None:
        n_blocks = max(need + 3, 4)
    assert ring_layer or need <= n_blocks
    p = make_params(H, Hkv, HD, dtype, bt, window=window, ring=ring, scale=scale, rows_per_tile=rows_per_tile, bidi=bidi)
    blk = bt * kvw
    if fill_unused:  # unwritten pages hold NaN patterns: nothing outside [0, P) may reach a result
        pool = np.full(n_blocks * 2 * blk, 0x7E00 if dtype == abi.ESP_F16 else 0x7FC0, np.uint16)
    else:
        pool = np.zeros(n_blocks * 2 * blk, np.uint16)
    perm = rng.permutation(n_blocks).astype(np.int32)
    n_rows = sum(M for _, M in seqs)
    Q = _bits(rng.standard_normal((n_rows, H * HD), dtype=np.float32) * sigma, dtype)
    Kb = _bits(rng.standard_normal((n_rows, kvw), dtype=np.float32) * sigma, dtype)
    Vb = _bits(rng.standard_normal((n_rows, kvw), dtype=np.float32) * sigma, dtype)
    trees = np.zeros(len(seqs), abi.TREE_DT)
    desc = np.zeros((n_rows, 4), np.int32)
    pos = np.zeros((n_rows, 4), np.int32)
    table = []
    base = 0
    used = 0
    for i, (P, M) in enumerate(seqs):
        nb = (P + bt - 1) // bt
        if ring_layer:
            tab0 = i * ring  # the slot's first ring block; key j lives in block (j / bt) % ring
            lo = max(0, P - ring * bt)  # older keys were overwritten
            K = _bits(rng.standard_normal((P - lo, kvw), dtype=np.float32) * sigma, dtype)
            V = _bits(rng.standard_normal((P - lo, kvw), dtype=np.float32) * sigma, dtype)
            for j in range(lo, P):
                b = tab0 + (j // bt) % ring
                pool[(2 * b) * blk + (j % bt) * kvw:(2 * b) * blk + (j % bt + 1) * kvw] = K[j - lo]
                pool[(2 * b + 1) * blk + (j % bt) * kvw:(2 * b + 1) * blk + (j % bt + 1) * kvw] = V[j - lo]
        else:
            tab0 = len(table)
            ids = perm[used:used + nb]
            used += nb
            table.extend(int(x) for x in ids)
            K = _bits(rng.standard_normal((nb * bt, kvw), dtype=np.float32) * sigma, dtype)
            V = _bits(rng.standard_normal((nb * bt, kvw), dtype=np.float32) * sigma, dtype)
            if fill_unused and P % bt:  # the tail of the last page was never written
                K[P:] = pool[0]
                V[P:] = pool[0]
            pv = pool.reshape(n_blocks, 2, bt, kvw)
            pv[ids, 0] = K.reshape(nb, bt, kvw)
            pv[ids, 1] = V.reshape(nb, bt, kvw)
        trees[i] = (base, P, tab0, M)
        pos[base:base + M, 0:3] = (P + np.arange(M))[:, None]
        if desc_fn is not None:
            desc[base:base + M] = desc_fn(M)
        base += M
    blocks = np.asarray(table if table else [0], np.int32)
    return Case(name, p, Q, Kb, Vb, pool, n_blocks, blocks, trees, desc, pos, n_rows,
                dict(seqs=list(seqs), seed=seed))


def make_prep(kind, H, Hkv, HD, dtype, n_rows, seed=0, bt=16, max_pos=40000):
    """Inputs of one esp_attn_prep call in the arrangement of one of the reference's three prep
    kernels: "qwen35" (kernels/40_attention.metal:9-102: a gate beside each query head, 64 rotating
    dims, position component per frequency), "gemma" (80_gemma.metal:52-108: all dims rotate by pos.x,
    values normalised), "omni" (82_qwen3_omni.metal:30-88: all dims rotate, component per frequency,
    queries scaled). Returns (params, dict of numpy arrays)."""
    rng = np.random.default_rng(seed)
    p = abi.PrepParams()
    p.H, p.Hkv, p.head_dim, p.dtype = H, Hkv, HD, dtype
    p.q_hs = 2 * HD if kind == "qwen35" else HD
    p.q_off = 0
    p.k_off = H * p.q_hs
    p.v_off = p.k_off + Hkv * HD
    p.x_ld = p.v_off + Hkv * HD
    p.q_ld, p.kv_ld = H * HD, Hkv * HD
    p.rope_dims = 64 if kind == "qwen35" else HD
    p.v_norm = 1 if kind == "gemma" else 0
    p.bt, p.eps = bt, 1e-6
    p.q_scale = float(1.0 / np.sqrt(HD)) if kind == "omni" else 1.0
    p.kv_base = 0
    half = p.rope_dims // 2
    a = dict(
        X=(rng.standard_normal((n_rows, p.x_ld), dtype=np.float32) * 1.5),
        qn_w=(1.0 + 0.25 * rng.standard_normal(HD, dtype=np.float32)),
        kn_w=(1.0 + 0.25 * rng.standard_normal(HD, dtype=np.float32)),
        inv_freq=(1.0e6 ** (-np.arange(half, dtype=np.float64) / half)).astype(np.float32),
        rope_sel=None if kind == "gemma" else (np.arange(half) % 3).astype(np.int32),
        pos=np.zeros((n_rows, 4), np.int32),
    )
    t = rng.integers(0, max_pos, n_rows)
    a["pos"][:, 0] = t
    a["pos"][:, 1] = t if kind == "gemma" else rng.integers(0, 64, n_rows)
    a["pos"][:, 2] = t if kind == "gemma" else rng.integers(0, 64, n_rows)
    return p, a


def make_gate(H, HD, D, dtype, n_rows, seed=0, q_ld=None, x_ld=None):
    """Inputs of one esp_head_gate call (sp_head_gate, kernels/85_spark.metal:96-128): O as an
    attention leaves it, the layer's normed input X and the gate rows Wg, as storage bits.
    Wg ~ N(0, 1) * 2 / sqrt(D) puts the dots at about N(0, 1): gates across the whole sigmoid."""
    rng = np.random.default_rng(seed)
    p = abi.GateParams()
    p.H, p.head_dim, p.D, p.dtype = H, HD, D, dtype
    p.q_ld = q_ld or H * HD
    p.x_ld = x_ld or D
    a = dict(
        O=_bits(rng.standard_normal((n_rows, p.q_ld), dtype=np.float32) * 0.5, dtype),
        X=_bits(rng.standard_normal((n_rows, p.x_ld), dtype=np.float32) * 0.5, dtype),
        Wg=_bits(rng.standard_normal((H, D), dtype=np.float32) * (2.0 / np.sqrt(D)), dtype),
    )
    return p, a


# ---- the five benchmark shapes, with a shrink factor for tests ----
def c1_single_decode(ctx=1024):
    return make_case("c1_single_decode", 1, 32, 4, 128, abi.ESP_F16, 16, [(ctx, 1)], rows_per_tile=1)


def c2_lengths(n_seqs=16, lo=512, hi=8192, seed=2):
    return [int(x) for x in np.random.default_rng(seed).integers(lo, hi + 1, n_seqs)]


def c2_batched_decode(n_seqs=16, lo=512, hi=8192, n_blocks=None):
    seqs = [(L, 1) for L in c2_lengths(n_seqs, lo, hi)]
    return make_case("c2_batched_decode", 2, 32, 4, 128, abi.ESP_F16, 16, seqs, n_blocks=n_blocks, rows_per_tile=1)


def c3_chunk(P, M=2048, n_blocks=None):
    return make_case(f"c3_prefill_P{P}", 3, 40, 8, 128, abi.ESP_BF16, 16, [(P, M)], n_blocks=n_blocks, rows_per_tile=128)


def c4_decode(sliding, n_seqs=8, ctx=16384, window=1024):
    return make_case("c4_decode_" + ("sliding" if sliding else "global"), 4, 16, 8, 256, abi.ESP_F16, 16,
                     [(ctx, 1)] * n_seqs, window=window if sliding else 0, rows_per_tile=1)


def c4_prefill(sliding, n_seqs=8, P=15360, M=1024, window=1024):
    return make_case("c4_prefill_" + ("sliding" if sliding else "global"), 4, 16, 8, 256, abi.ESP_F16, 16,
                     [(P, M)] * n_seqs, window=window if sliding else 0, rows_per_tile=128)


def c5_verify(n_seqs=8, ctx=32768, drafts=4):
    return make_case("c5_verify", 5, 32, 4, 128, abi.ESP_F16, 16, [(ctx, drafts)] * n_seqs, rows_per_tile=drafts,
                     desc_fn=lambda M: verify_desc(M, 1))
