"""Calls into libespetero_attn.so with torch tensors as device memory.

torch is plumbing here (allocation, streams, host<->device copies); every
computation happens behind the C ABI. There is no fallback path: a missing or
failing library raises.
"""
import ctypes as C

import numpy as np
import torch

from . import abi

_ERRLEN = 512


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream(stream):
    if stream is None:
        stream = torch.cuda.current_stream()
    return C.c_void_p(stream.cuda_stream)


def init(device=0):
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_attn_init(device, err, _ERRLEN), err)


def to_dev(a, device="cuda"):
    """numpy array (any dtype, incl. structured records) -> device tensor of raw bytes / ints."""
    a = np.ascontiguousarray(a)
    if a.dtype.fields is not None or a.dtype == np.uint16:
        flat = a.view(np.uint8).reshape(-1)
        return torch.from_numpy(flat.copy()).to(device)
    return torch.from_numpy(a.copy()).to(device)


def plan_hint(params, device=0):
    """(workgroups resident at once, workgroups per tile) of the kernel serving `params`:
    the planner's split target and its `groups` argument."""
    return plan_hint3(params, device)[:2]


def plan_hint3(params, device=0):
    """plan_hint plus the largest rows_per_tile the tiled kernel takes at this head_dim."""
    err = C.create_string_buffer(_ERRLEN)
    n, g, r = C.c_int32(0), C.c_int32(0), C.c_int32(0)
    abi.check(abi.attn_lib().esp_attn_plan_hint(C.byref(params), device, C.byref(n), C.byref(g), C.byref(r), err, _ERRLEN), err)
    return n.value, g.value, r.value


def workspace_bytes(params, n_rows, n_parts):
    return abi.attn_lib().esp_attn_workspace_bytes(C.byref(params), n_rows, n_parts)


def forward(params, Q, Kb, Vb, pool, blocks, desc, pos, O, tiles, n_tiles, trees, n_trees, jobs, n_jobs, n_parts, n_rows,
            workspace, stream=None):
    """All tensors are device tensors (records as byte tensors). Enqueues on `stream`."""
    err = C.create_string_buffer(_ERRLEN)
    rc = abi.attn_lib().esp_attn_forward(
        C.byref(params), _ptr(Q), _ptr(Kb), _ptr(Vb), _ptr(pool), _ptr(blocks), _ptr(desc), _ptr(pos), _ptr(O),
        _ptr(tiles), n_tiles, _ptr(trees), n_trees, _ptr(jobs), n_jobs, n_parts, n_rows, _ptr(workspace),
        0 if workspace is None else workspace.numel() * workspace.element_size(), _stream(stream), err, _ERRLEN)
    abi.check(rc, err)


def forward_static(params, Q, Kb, Vb, pool, blocks, desc, pos, O, tiles, n_tiles, trees, n_trees, jobs, n_jobs, n_parts, n_rows,
                   stream=None):
    """forward() over the library's own scratch array: no workspace, no allocation."""
    err = C.create_string_buffer(_ERRLEN)
    rc = abi.attn_lib().esp_attn_forward_static(
        C.byref(params), _ptr(Q), _ptr(Kb), _ptr(Vb), _ptr(pool), _ptr(blocks), _ptr(desc), _ptr(pos), _ptr(O),
        _ptr(tiles), n_tiles, _ptr(trees), n_trees, _ptr(jobs), n_jobs, n_parts, n_rows, _stream(stream), err, _ERRLEN)
    abi.check(rc, err)


def validate(params, tiles, trees, jobs, n_parts, n_rows, blocks, pool_blocks, fused=False, rows_in_pool=False):
    """Host-side bounds check of a pass's records (numpy arrays) before they are uploaded. Raises EspError.
    fused: the pass goes to esp_attn_decode_fused (also: one tile group per tree, trees of at most rows_per_tile rows).
    rows_in_pool: the pass runs without Kb / Vb (also: block lists that reach P + M, P - base a multiple of 16 on the tiled kernel)."""
    tiles = np.ascontiguousarray(tiles, dtype=abi.TILE_DT)
    trees = np.ascontiguousarray(trees, dtype=abi.TREE_DT)
    jobs = np.ascontiguousarray(jobs, dtype=abi.COMBINE_DT)
    blocks = None if blocks is None else np.ascontiguousarray(blocks, dtype=np.int32)
    hp = lambda a: None if a is None or a.size == 0 else a.ctypes.data  # noqa: E731
    err = C.create_string_buffer(_ERRLEN)
    mode = (abi.ESP_PASS_FUSED if fused else 0) | (abi.ESP_PASS_ROWS_IN_POOL if rows_in_pool else 0)
    rc = abi.attn_lib().esp_attn_validate_for(C.byref(params), mode, hp(tiles), len(tiles), hp(trees), len(trees), hp(jobs), len(jobs),
                                              n_parts, n_rows, hp(blocks), 0 if blocks is None else len(blocks), pool_blocks, err, _ERRLEN)
    abi.check(rc, err)


def time_next(start, stop):
    """The next forward() records its attention kernel's begin and end into these two torch events
    (created with enable_timing=True and recorded once before, so that their handles exist)."""
    rc = abi.attn_lib().esp_attn_time_next(C.c_void_p(start.cuda_event), C.c_void_p(stop.cuda_event))
    if rc != 0:
        raise abi.EspError(f"esp_attn_time_next: error {rc}")


def combine(params, O, jobs, n_jobs, n_parts, n_rows, workspace, stream=None):
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_attn_combine(C.byref(params), _ptr(O), _ptr(jobs), n_jobs, n_parts, n_rows, _ptr(workspace),
                                              workspace.numel() * workspace.element_size(), _stream(stream), err, _ERRLEN), err)


def kv_save(params, Kb, Vb, pool, entries, n_entries, stream=None):
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_kv_save(C.byref(params), _ptr(Kb), _ptr(Vb), _ptr(pool), _ptr(entries), n_entries,
                                         _stream(stream), err, _ERRLEN), err)


def kv_copy_blocks(params, pool, pairs, n_pairs, n_layers, region_elems, stream=None):
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_kv_copy_blocks(C.byref(params), _ptr(pool), _ptr(pairs), n_pairs, n_layers,
                                                C.c_uint64(region_elems), _stream(stream), err, _ERRLEN), err)


def kv_gather(params, pool, blocks, n_tokens, K_out, V_out, stream=None):
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_kv_gather(C.byref(params), _ptr(pool), _ptr(blocks), n_tokens, _ptr(K_out), _ptr(V_out),
                                           _stream(stream), err, _ERRLEN), err)


def kv_relayout(params, src, src_layout, dst, dst_layout, n_blocks, stream=None):
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_kv_relayout(C.byref(params), _ptr(src), src_layout, _ptr(dst), dst_layout, n_blocks,
                                             _stream(stream), err, _ERRLEN), err)


def kv_export_blocks(params, pool, blocks, n_blocks, out, stream=None):
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_kv_export_blocks(C.byref(params), _ptr(pool), _ptr(blocks), n_blocks, _ptr(out),
                                                  _stream(stream), err, _ERRLEN), err)


def kv_import_blocks(params, src, blocks, n_blocks, pool, stream=None):
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_kv_import_blocks(C.byref(params), _ptr(src), _ptr(blocks), n_blocks, _ptr(pool),
                                                  _stream(stream), err, _ERRLEN), err)


def attn_prep(params, X, qn_w, kn_w, pos, inv_freq, rope_sel, Q, Kb, Vb, row_table, pool, n_rows, stream=None):
    """All device tensors; rope_sel, row_table and pool may be None."""
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_attn_prep(C.byref(params), _ptr(X), _ptr(qn_w), _ptr(kn_w), _ptr(pos), _ptr(inv_freq),
                                           _ptr(rope_sel), _ptr(Q), _ptr(Kb), _ptr(Vb), _ptr(row_table), _ptr(pool), n_rows,
                                           _stream(stream), err, _ERRLEN), err)


def decode_fused(pp, params, X, qn_w, kn_w, pos, inv_freq, rope_sel, row_table, pool, dp, O, stream=None):
    """attn_prep fused into the attention of a decode / short verify pass. dp: the DevicePass holding the records."""
    err = C.create_string_buffer(_ERRLEN)
    ws = dp.workspace
    abi.check(abi.attn_lib().esp_attn_decode_fused(
        C.byref(pp), C.byref(params), _ptr(X), _ptr(qn_w), _ptr(kn_w), _ptr(pos), _ptr(inv_freq), _ptr(rope_sel), _ptr(row_table),
        _ptr(pool), _ptr(dp.blocks), _ptr(dp.desc), _ptr(O), _ptr(dp.tiles), dp.n_tiles, _ptr(dp.trees), dp.n_trees, _ptr(dp.jobs),
        dp.n_jobs, dp.n_parts, dp.n_rows, _ptr(ws), ws.numel() * ws.element_size(), _stream(stream), err, _ERRLEN), err)


def head_gate(params, O, X, Wg, dots, n_rows, stream=None):
    """Device tensors. O (gated in place) or dots (fp32 [n_rows][H], written) may be None, not both."""
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_head_gate(C.byref(params), _ptr(O), _ptr(X), _ptr(Wg), _ptr(dots), n_rows,
                                           _stream(stream), err, _ERRLEN), err)


def chain_advance(trees, n_trees, pos, row_table, blocks, bt, ring=0, stream=None):
    """Device tensors: trees (TREE_DT bytes), pos / row_table int32 [rows][4], blocks int32."""
    err = C.create_string_buffer(_ERRLEN)
    abi.check(abi.attn_lib().esp_chain_advance(_ptr(trees), n_trees, _ptr(pos), _ptr(row_table), _ptr(blocks), bt, ring,
                                               _stream(stream), err, _ERRLEN), err)


class DevicePass:
    """One planned pass resident on the device: uploads the records once and
    replays esp_attn_forward (what a decode chain does between host syncs)."""

    def __init__(self, params, trees, tiles, jobs, n_parts, n_rows, blocks, desc=None, pos=None, device="cuda",
                 pool_blocks=None, static=False, fused=False, rows_in_pool=False):
        """pool_blocks: blocks in the pool; when given, the records are checked on the host before the upload
        (fused: with the checks of a pass meant for decode_fused).
        static: run over the library's own scratch array (esp_attn_forward_static) instead of a workspace."""
        if pool_blocks is not None:
            validate(params, tiles, trees, jobs, n_parts, n_rows, blocks, pool_blocks, fused=fused, rows_in_pool=rows_in_pool)
        self.params = params
        self.static = static
        self.n_trees, self.n_tiles, self.n_jobs = len(trees), len(tiles), len(jobs)
        self.n_parts, self.n_rows = n_parts, n_rows
        self.trees_host, self.tiles_host, self.jobs_host = trees, tiles, jobs
        self.trees = to_dev(np.ascontiguousarray(trees, dtype=abi.TREE_DT), device)
        self.tiles = to_dev(np.ascontiguousarray(tiles, dtype=abi.TILE_DT), device)
        self.jobs = to_dev(np.ascontiguousarray(jobs, dtype=abi.COMBINE_DT), device) if len(jobs) else None
        self.blocks = to_dev(np.ascontiguousarray(blocks, dtype=np.int32), device) if blocks is not None else None
        self.desc = to_dev(np.ascontiguousarray(desc, dtype=np.int32), device) if desc is not None else None
        self.pos = to_dev(np.ascontiguousarray(pos, dtype=np.int32), device) if pos is not None else None
        nbytes = workspace_bytes(params, n_rows, n_parts)
        self.workspace = None if static else torch.empty(nbytes, dtype=torch.uint8, device=device)
        self._key, self._fn, self._args, self._err = None, None, None, C.create_string_buffer(_ERRLEN)

    def run(self, Q, Kb, Vb, pool, O, stream=None, merge=True):
        """Enqueues the pass. The ctypes argument list is built once per set of buffers and reused: a decode step is
        tens of microseconds on the GPU, and rebuilding twenty pointer objects per call costs the host as much."""
        st = torch.cuda.current_stream().cuda_stream if stream is None else stream.cuda_stream
        key = (Q.data_ptr(), None if Kb is None else Kb.data_ptr(), None if Vb is None else Vb.data_ptr(), pool.data_ptr(), O.data_ptr(), st, merge,
               None if self.pos is None else self.pos.data_ptr())
        if self._key != key:
            jobs, n_jobs = (self.jobs, self.n_jobs) if merge else (None, 0)
            head = [C.byref(self.params), _ptr(Q), _ptr(Kb), _ptr(Vb), _ptr(pool), _ptr(self.blocks), _ptr(self.desc), _ptr(self.pos),
                    _ptr(O), _ptr(self.tiles), self.n_tiles, _ptr(self.trees), self.n_trees, _ptr(jobs), n_jobs, self.n_parts, self.n_rows]
            if self.static:
                self._fn, self._args = abi.attn_lib().esp_attn_forward_static, head + [C.c_void_p(st), self._err, _ERRLEN]
            else:
                ws = self.workspace
                self._fn = abi.attn_lib().esp_attn_forward
                self._args = head + [_ptr(ws), ws.numel() * ws.element_size(), C.c_void_p(st), self._err, _ERRLEN]
            self._key = key
        rc = self._fn(*self._args)
        if rc:
            abi.check(rc, self._err)

    def merge(self, O, stream=None):
        if self.n_jobs:
            combine(self.params, O, self.jobs, self.n_jobs, self.n_parts, self.n_rows, self.workspace, stream)
