"""ctypes binding of the CPU checker (oracle/attn_oracle.c) plus a float64
brute force. TEST INFRASTRUCTURE: imported only by tests/, the smoke check
and the bench's cpu_baseline leg; the product never touches it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from espetero_amd import abi

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "libattn_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-s", "-C", _DIR, "-B"], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.esp_oracle_h2f.restype = C.c_float
        L.esp_oracle_h2f.argtypes = [C.c_uint16]
        L.esp_oracle_f2h.restype = C.c_uint16
        L.esp_oracle_f2h.argtypes = [C.c_float]
        L.esp_oracle_bf2f.restype = C.c_float
        L.esp_oracle_bf2f.argtypes = [C.c_uint16]
        L.esp_oracle_f2bf.restype = C.c_uint16
        L.esp_oracle_f2bf.argtypes = [C.c_float]
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


TOL = 2e-3  # max-abs contract of the path (fp32 accumulation, fp16 / bf16 storage)


def bf16_ulp(x):
    """One unit in the last place of a bf16 number of x's magnitude: 8 significant bits, 2^(floor(log2 |x|) - 7)."""
    ax = np.maximum(np.abs(np.asarray(x, np.float64)), 2.0 ** -126)
    return 2.0 ** (np.floor(np.log2(ax)) - 7)


def beyond_rounding(got, want, dtype, want_rounded):
    """Largest |got - want| once the rounding of the stored output itself is taken off: nothing for fp16 (half a unit
    in the last place of an output below 1 is 2.4e-4, inside the bar), and for bf16 half a unit in the last place
    against an unrounded expectation, a whole unit against one that was itself rounded to bf16 (two results a hair
    apart may round to neighbouring bf16 numbers). The one bar every comparison of this path uses is TOL on this."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64).reshape(np.shape(got))
    allow = 0.0 if dtype == abi.ESP_F16 else bf16_ulp(np.maximum(np.abs(got), np.abs(want))) * (1.0 if want_rounded else 0.5)
    return float(np.maximum(np.abs(got - want) - allow, 0.0).max())


def _u16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16
    return a


def _i32(a):
    if a is None:
        return None
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a


def attn_direct(params, Q, Kb, Vb, pool, blocks, desc, pos, trees, n_threads=1):
    """Row-by-row semantics. Q/Kb/Vb/pool: uint16 storage bits. Returns O (uint16)."""
    Q, Kb, Vb, pool = _u16(Q), _u16(Kb), _u16(Vb), _u16(pool)
    blocks, desc, pos = _i32(blocks), _i32(desc), _i32(pos)
    trees = np.ascontiguousarray(trees, dtype=abi.TREE_DT)
    O = np.zeros_like(Q)
    rc = lib().esp_oracle_attn_direct(C.byref(params), _p(Q), _p(Kb), _p(Vb), _p(pool), _p(blocks), _p(desc), _p(pos),
                                      _p(O), _p(trees), C.c_int(len(trees)), C.c_int(n_threads))
    assert rc == 0
    return O


def attn_tiles(params, Q, Kb, Vb, pool, blocks, desc, pos, tiles, trees, jobs, n_parts):
    """Through tiles, partial records and the merge, as the reference kernels are structured."""
    Q, Kb, Vb, pool = _u16(Q), _u16(Kb), _u16(Vb), _u16(pool)
    blocks, desc, pos = _i32(blocks), _i32(desc), _i32(pos)
    trees = np.ascontiguousarray(trees, dtype=abi.TREE_DT)
    tiles = np.ascontiguousarray(tiles, dtype=abi.TILE_DT)
    jobs = np.ascontiguousarray(jobs, dtype=abi.COMBINE_DT)
    G = params.H // params.Hkv
    parts = np.zeros(max(1, n_parts) * params.Hkv * params.rows_per_tile * G * (params.head_dim + 2), np.float32)
    O = np.zeros_like(Q)
    rc = lib().esp_oracle_attn_tiles(C.byref(params), _p(Q), _p(Kb), _p(Vb), _p(pool), _p(blocks), _p(desc), _p(pos),
                                     _p(O), _p(tiles), C.c_int(len(tiles)), _p(trees), C.c_int(len(trees)), _p(jobs),
                                     C.c_int(len(jobs)), _p(parts))
    assert rc == 0
    return O


def kv_save(params, Kb, Vb, pool, entries):
    entries = np.ascontiguousarray(entries, dtype=abi.KVSAVE_DT)
    lib().esp_oracle_kv_save(C.byref(params), _p(_u16(Kb)), _p(_u16(Vb)), _p(pool), _p(entries), C.c_int(len(entries)))


def kv_copy_blocks(params, pool, pairs, n_layers, region_elems):
    pairs = np.ascontiguousarray(pairs, dtype=np.int32).reshape(-1, 2)
    lib().esp_oracle_kv_copy_blocks(C.byref(params), _p(pool), _p(pairs), C.c_int(len(pairs)), C.c_int(n_layers),
                                    C.c_uint64(region_elems))


def kv_gather(params, pool, blocks, n_tokens):
    w = params.Hkv * params.head_dim
    K = np.zeros((n_tokens, w), np.uint16)
    V = np.zeros((n_tokens, w), np.uint16)
    blocks = _i32(blocks)
    lib().esp_oracle_kv_gather(C.byref(params), _p(_u16(pool)), _p(blocks), C.c_int(n_tokens), _p(K), _p(V))
    return K, V


def attn_prep(params, X, qn_w, kn_w, pos, inv_freq, rope_sel, n_rows, row_table=None, pool=None):
    """Returns Q, Kb, Vb as storage bits; writes the folded append into `pool` (reference layout) in place."""
    Q = np.zeros((n_rows, params.q_ld), np.uint16)
    Kb = np.zeros((n_rows, params.kv_ld), np.uint16)
    Vb = np.zeros((n_rows, params.kv_ld), np.uint16)
    f32 = lambda a: None if a is None else np.ascontiguousarray(a, dtype=np.float32)  # noqa: E731
    X, qn_w, kn_w, inv_freq = f32(X), f32(qn_w), f32(kn_w), f32(inv_freq)
    pos, rope_sel, row_table = _i32(pos), _i32(rope_sel), _i32(row_table)
    lib().esp_oracle_attn_prep(C.byref(params), _p(X), _p(qn_w), _p(kn_w), _p(pos), _p(inv_freq), _p(rope_sel), _p(Q), _p(Kb),
                               _p(Vb), _p(row_table), _p(pool), C.c_int(n_rows))
    return Q, Kb, Vb


def head_gate(params, O, X, Wg, n_rows, want_dots=False):
    """sp_head_gate on storage bits: returns the gated copy of O (None when O is None) and, if asked, the fp32 dots."""
    out = None if O is None else np.array(_u16(O), copy=True)
    dots = np.zeros((n_rows, params.H), np.float32) if want_dots else None
    lib().esp_oracle_head_gate(C.byref(params), _p(out), _p(_u16(X)), _p(_u16(Wg)), _p(dots), C.c_int(n_rows))
    return (out, dots) if want_dots else out


def head_gate_f64(params, O, X, Wg, n_rows):
    """The closed form in float64, no second rounding: float(O) * sigmoid(x . Wg[h]); also returns the dots."""
    x = to_f32(np.asarray(X)[:, :params.D], params.dtype).astype(np.float64)
    w = to_f32(np.asarray(Wg), params.dtype).astype(np.float64).reshape(params.H, params.D)
    dots = x @ w.T
    g = 1.0 / (1.0 + np.exp(-dots))
    o = to_f32(np.asarray(O)[:, :params.H * params.head_dim], params.dtype).astype(np.float64)
    o = o.reshape(n_rows, params.H, params.head_dim) * g[:, :, None]
    return o, dots


def attn_prep_f64(params, X, qn_w, kn_w, pos, inv_freq, rope_sel, n_rows):
    """The closed forms in float64, no storage rounding: RMSNorm x / sqrt(mean x^2 + eps) * w, the rotation
    [[c, -s], [s, c]] on each pair (d, d + rope_dims / 2) by angle position * inv_freq, the query scale.
    The angle is formed in fp32 as the kernels form it (a float64 angle would be a different function of
    the integer position once position * inv_freq no longer fits 24 bits)."""
    p = params
    HD, half = p.head_dim, p.rope_dims // 2
    X = np.asarray(X, np.float64).reshape(n_rows, p.x_ld)
    Q = np.zeros((n_rows, p.H, HD))
    K = np.zeros((n_rows, p.Hkv, HD))
    V = np.zeros((n_rows, p.Hkv, HD))
    pos = np.asarray(pos, np.int64).reshape(n_rows, 4)
    sel = np.zeros(half, np.int64) if rope_sel is None else np.asarray(rope_sel, np.int64)[:half]
    ang = (pos[:, sel].astype(np.float32) * np.asarray(inv_freq, np.float32)[None, :half]).astype(np.float64)  # [rows][half]
    c, s = np.cos(ang), np.sin(ang)

    def norm(x):
        return x / np.sqrt((x * x).mean(-1, keepdims=True) + np.float64(np.float32(p.eps)))

    def rot(x):  # x [rows][heads][HD]
        y = x.copy()
        a, b = x[..., :half], x[..., half:2 * half]
        y[..., :half] = a * c[:, None, :] - b * s[:, None, :]
        y[..., half:2 * half] = b * c[:, None, :] + a * s[:, None, :]
        return y

    for h in range(p.H):
        Q[:, h] = X[:, p.q_off + h * p.q_hs:p.q_off + h * p.q_hs + HD]
    for h in range(p.Hkv):
        K[:, h] = X[:, p.k_off + h * HD:p.k_off + (h + 1) * HD]
        V[:, h] = X[:, p.v_off + h * HD:p.v_off + (h + 1) * HD]
    Q = rot(norm(Q) * np.asarray(qn_w, np.float64)) * np.float64(np.float32(p.q_scale))
    K = rot(norm(K) * np.asarray(kn_w, np.float64))
    if p.v_norm:
        V = norm(V)
    return Q.reshape(n_rows, -1), K.reshape(n_rows, -1), V.reshape(n_rows, -1)


# ---- storage conversions (numpy side) ----
def to_f32(bits, dtype):
    bits = np.asarray(bits, dtype=np.uint16)
    if dtype == abi.ESP_BF16:
        return (bits.astype(np.uint32) << 16).view(np.float32)
    return bits.view(np.float16).astype(np.float32)


def from_f32(x, dtype):
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dtype == abi.ESP_BF16:
        u = x.view(np.uint32)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return x.astype(np.float16).view(np.uint16)


# ---- float64 brute force: dense mask, no paging, no online softmax ----
def visible_mask(params, tree, desc, pos):
    """bool [M][P + M]: row rr of the tree sees cached key j (col j) / batch key j (col P + j).
    The textual rule at kernels/40_attention.metal:104-113 and 80_gemma.metal:283-285."""
    base, P, M = int(tree["base"]), int(tree["P"]), int(tree["M"])
    vis = np.zeros((M, P + M), bool)
    for rr in range(M):
        row = base + rr
        d = desc[row] if desc is not None else (0, 0, 0, 0)
        qpos = pos[row][0] if pos is not None else 0
        for j in range(P):
            vis[rr, j] = (qpos - j < params.window) if params.window > 0 else True
        for j in range(M):
            v = (j < d[2]) or (j >= d[0] and (j <= rr or (params.bidi and j < d[3])))
            if params.window > 0 and v:
                v = qpos - pos[base + j][0] < params.window
            vis[rr, P + j] = v
    return vis


def gather_tree_kv(params, tree, pool, blocks, Kb, Vb):
    """K, V float64 [P + M][Hkv][HD] of one tree (cached via the reference-layout pool, then batch)."""
    base, P, M, table = int(tree["base"]), int(tree["P"]), int(tree["M"]), int(tree["table"])
    HD, Hkv, bt, kv_ld = params.head_dim, params.Hkv, params.bt, params.kv_ld
    K = np.zeros((P + M, Hkv, HD), np.float64)
    V = np.zeros((P + M, Hkv, HD), np.float64)
    blk = bt * kv_ld
    for j in range(P):
        b = table + (j // bt) % params.ring if params.ring else int(blocks[table + j // bt])
        for which, out in ((0, K), (1, V)):
            a = params.kv_base + (2 * b + which) * blk + (j % bt) * kv_ld
            out[j] = to_f32(pool[a:a + Hkv * HD], params.dtype).reshape(Hkv, HD)
    for j in range(M):
        K[P + j] = to_f32(Kb[base + j, :Hkv * HD], params.dtype).reshape(Hkv, HD)
        V[P + j] = to_f32(Vb[base + j, :Hkv * HD], params.dtype).reshape(Hkv, HD)
    return K, V


def brute_force(params, Q, Kb, Vb, pool, blocks, desc, pos, trees, gate=None):
    """O in float64, [n_rows][H][HD]; rows of no tree stay 0. No rounding of P."""
    HD, H, Hkv = params.head_dim, params.H, params.Hkv
    G = H // Hkv
    n_rows = Q.shape[0]
    O = np.zeros((n_rows, H, HD), np.float64)
    for tree in trees:
        base, P, M = int(tree["base"]), int(tree["P"]), int(tree["M"])
        K, V = gather_tree_kv(params, tree, pool, blocks, Kb, Vb)
        vis = visible_mask(params, tree, desc, pos)
        q = to_f32(Q[base:base + M, :H * HD], params.dtype).astype(np.float64).reshape(M, H, HD)
        for h in range(H):
            kvh = h // G
            s = (q[:, h, :] @ K[:, kvh, :].T) * float(params.scale)
            s = np.where(vis, s, -np.inf)
            m = s.max(axis=1, keepdims=True)
            m = np.where(np.isfinite(m), m, 0.0)
            p = np.exp(s - m)
            l = p.sum(axis=1, keepdims=True)
            o = p @ V[:, kvh, :]
            o = np.where(l > 0, o / np.where(l > 0, l, 1.0), 0.0)
            if gate is not None:
                o = o / (1.0 + np.exp(-gate[base:base + M, h, :].astype(np.float64)))
            O[base:base + M, h, :] = o
    return O
