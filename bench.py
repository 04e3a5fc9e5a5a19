#!/usr/bin/env python3
"""Paged-KV attention benchmark on one MI355X.

A step is one pass of the hot path over one batch of synthetic input, through
the C ABI, inputs resident in HBM when the clock starts. The default workload
is the batched paged decode (16 sequences, contexts uniform in [512, 8192],
32 Q / 4 KV heads, head_dim 128, fp16, page 16, pages scattered over a shared
64K-page pool); --workload picks the other benchmark shapes.

Prints ONE JSON line: whole-job throughput (`value`), the roofline of the
dominant kernel measured with HIP events on the launch stream, and the CPU
checker timed on a bounded sample of the same workload on the host cores.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0    # dense fp16 / bf16
N_CU = 256


class Workload:
    """Device-resident inputs of one benchmark shape plus the planned passes."""

    def __init__(self, name, H, Hkv, HD, dtype, bt, seqs, window=0, rows_per_tile=1, desc_fn=None, pool_pages=65536,
                 seed=0, workgroups=None, bound="hbm", contiguous=False, rows_in_pool=None):
        import torch
        from espetero_amd import abi, device, host, synth
        self.torch, self.abi, self.device, self.host = torch, abi, device, host
        self.name, self.bound, self.dtype = name, bound, dtype
        self.H, self.Hkv, self.HD, self.bt, self.window = H, Hkv, HD, bt, window
        self.seqs = list(seqs)
        p = synth.make_params(H, Hkv, HD, dtype, bt, window=window, rows_per_tile=rows_per_tile)
        if rows_per_tile > 32:  # a prefill pass: plan with the largest tile the tiled kernel takes
            rows_per_tile = device.plan_hint3(p)[2]
            p.rows_per_tile = rows_per_tile
        self.params = p
        tdt = torch.float16 if dtype == abi.ESP_F16 else torch.bfloat16
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        page_elems = 2 * bt * Hkv * HD
        pages_per_set = sum((P + M + bt - 1) // bt for P, M in self.seqs)
        self.n_sets = max(1, min(16, pool_pages // max(pages_per_set, 1)))
        self.pool_pages = max(pool_pages, pages_per_set)
        # The pool holds N(0, 1) * 0.5 everywhere: any page is a valid K / V page in the native layout.
        self.pool = torch.empty(self.pool_pages * page_elems, dtype=tdt, device="cuda")
        chunk = 1 << 26
        for s in range(0, self.pool.numel(), chunk):
            n = min(chunk, self.pool.numel() - s)
            self.pool[s:s + n] = (torch.randn(n, generator=g, device="cuda", dtype=torch.float32) * 0.5).to(tdt)
        n_rows = sum(M for _, M in self.seqs)
        self.n_rows = n_rows
        self.Q = (torch.randn(n_rows, H * HD, generator=g, device="cuda") * 0.5).to(tdt)
        self.Kb = (torch.randn(n_rows, Hkv * HD, generator=g, device="cuda") * 0.5).to(tdt)
        self.Vb = (torch.randn(n_rows, Hkv * HD, generator=g, device="cuda") * 0.5).to(tdt)
        self.O = torch.zeros_like(self.Q)
        # rows, trees, descriptors
        trees = np.zeros(len(self.seqs), abi.TREE_DT)
        desc = np.zeros((n_rows, 4), np.int32)
        pos = np.zeros((n_rows, 4), np.int32)
        base, tab = 0, 0
        for i, (P, M) in enumerate(self.seqs):
            trees[i] = (base, P, tab, M)
            pos[base:base + M, :3] = (P + np.arange(M))[:, None]
            if desc_fn is not None:
                desc[base:base + M] = desc_fn(M)
            base += M
            tab += (P + M + bt - 1) // bt
        self.trees, self.desc, self.pos = trees, desc, pos
        resident, groups = device.plan_hint(p)
        opts = host.options_mi355x(rows_per_tile, workgroups or resident)
        for k, v in PLAN_TWEAK.items():   # experiments from the command line (--cut-batch, --plan-costs)
            setattr(opts, k, v)
        self.tiles, self.jobs, self.n_parts = host.plan_tiles(trees, groups, window, pos if window > 0 else None, opts)
        # Block tables: disjoint slices of one seeded permutation of the pool, one slice per
        # rotation set, so a step never finds the previous step's pages in a cache.
        perm = np.random.default_rng(seed + 1).permutation(self.pool_pages).astype(np.int32)
        if contiguous:  # experiment: pages in address order
            perm = np.arange(self.pool_pages, dtype=np.int32)
        self.tables = [perm[s * pages_per_set:(s + 1) * pages_per_set].copy() for s in range(self.n_sets)]
        # Prefill passes read their own rows from the pool (esp_attn_forward without Kb / Vb): the rows are appended
        # once, here, to positions P + j of every rotation set's block lists, as esp_attn_prep with a row table leaves
        # them in front of the attention of a layer. Decode and verify passes hand their rows over as Kb / Vb.
        self.rows_in_pool = (rows_per_tile > 32) if rows_in_pool is None else rows_in_pool
        self.passes = [device.DevicePass(p, trees, self.tiles, self.jobs, self.n_parts, n_rows, t,
                                         desc if desc_fn is not None else None, pos if window > 0 else None,
                                         pool_blocks=self.pool_pages, rows_in_pool=self.rows_in_pool)
                       for t in self.tables]
        if self.rows_in_pool:
            e = np.zeros(n_rows, abi.KVSAVE_DT)
            e["src_row"] = np.arange(n_rows)
            for t in self.tables:
                for tr in trees:
                    b0, P, tab, M = int(tr["base"]), int(tr["P"]), int(tr["table"]), int(tr["M"])
                    q = P + np.arange(M)
                    e["block"][b0:b0 + M], e["pos"][b0:b0 + M] = t[tab + q // bt], q % bt
                device.kv_save(p, self.Kb, self.Vb, self.pool, device.to_dev(e), n_rows)
            torch.cuda.synchronize()
        # algorithmic work: every visible K and V element once + Q + O + block-table entries; visible (q, k) pairs
        es = 2
        vis_keys, pairs = 0, 0
        for P, M in self.seqs:
            for r in range(M):
                lo = max(0, P + r - window + 1) if window > 0 else 0
                pairs += (P + r + 1) - lo
            lo = max(0, P - window + 1) if window > 0 else 0
            vis_keys += (P + M) - lo
        self.alg_bytes = vis_keys * Hkv * HD * 2 * es + 2 * n_rows * H * HD * es + ((vis_keys + bt - 1) // bt) * 4
        self.alg_flops = 4 * HD * H * pairs

    def step(self, i, merge=True):
        """Enqueue one pass: attention + split-K merge, one call."""
        dp = self.passes[i % self.n_sets]
        if self.rows_in_pool:
            dp.run(self.Q, None, None, self.pool, self.O, merge=merge)
        else:
            dp.run(self.Q, self.Kb, self.Vb, self.pool, self.O, merge=merge)

    def launch(self, i, l=0):
        """The pass's dominant kernel alone: the attention without the merge that follows it."""
        self.step(i, merge=False)


class PrepWorkload:
    """esp_attn_prep over one chunk of rows: fp32 fused projection in, Q / K / V in the storage type out,
    the rows' K / V appended to a paged pool by the same kernel."""

    kernel = "attn_prep_kernel"

    def __init__(self, name, kind, H, Hkv, HD, dtype, n_rows, bt=16, seed=7):
        import torch
        from espetero_amd import abi, device, synth
        self.torch, self.device = torch, device
        self.name, self.bound, self.dtype = name, "hbm", dtype
        self.H, self.Hkv, self.HD, self.bt, self.window = H, Hkv, HD, bt, 0
        self.seqs, self.n_rows, self.tiles, self.n_parts = [(0, n_rows)], n_rows, [], 0
        self.kind = kind
        p, a = synth.make_prep(kind, H, Hkv, HD, dtype, n_rows, seed=seed, bt=bt)
        self.params, self.host = p, a
        tdt = torch.float16 if dtype == abi.ESP_F16 else torch.bfloat16
        dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
        # rotation sets of X so that a step never finds its input in a cache
        self.n_sets = 4
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        self.X = [dev(a["X"])] + [torch.randn(n_rows, p.x_ld, generator=g, device="cuda") * 1.5 for _ in range(self.n_sets - 1)]
        self.qn_w, self.kn_w, self.pos = dev(a["qn_w"]), dev(a["kn_w"]), dev(a["pos"])
        self.inv_freq, self.rope_sel = dev(a["inv_freq"]), dev(a["rope_sel"])
        self.Q = torch.zeros(n_rows, p.q_ld, dtype=tdt, device="cuda")
        self.Kb = torch.zeros(n_rows, p.kv_ld, dtype=tdt, device="cuda")
        self.Vb = torch.zeros_like(self.Kb)
        n_blocks = (n_rows + bt - 1) // bt
        self.pool_pages = n_blocks
        self.pool = torch.zeros(n_blocks * 2 * bt * p.kv_ld, dtype=tdt, device="cuda")
        perm = np.random.default_rng(seed).permutation(n_blocks).astype(np.int32)
        table = np.full((n_rows, 4), -1, np.int32)
        table[:, 0] = perm[np.arange(n_rows) // bt]
        table[:, 1] = np.arange(n_rows) % bt
        self.table_host, self.table = table, dev(table)
        elems = (H + 2 * Hkv) * HD
        self.alg_bytes = n_rows * (elems * 4 + elems * 2 + 2 * Hkv * HD * 2 + 16 + 16)  # X, Q K V, pool entries, pos, table
        self.alg_flops = 0

    def step(self, i):
        self.device.attn_prep(self.params, self.X[i % self.n_sets], self.qn_w, self.kn_w, self.pos, self.inv_freq, self.rope_sel,
                              self.Q, self.Kb, self.Vb, self.table, self.pool, self.n_rows)

    def launch(self, i, l=0):
        self.step(i)


class GateWorkload:
    """esp_head_gate over the rows of one prefill pass: O *= sigmoid(x . Wg[h]) in place (the reference's
    form), or with dots_only the fp32 dots alone, which the attention's own epilogue then applies."""

    kernel = "head_gate_kernel"

    def __init__(self, name, H, HD, D, dtype, n_rows, dots_only=False, seed=9):
        import torch
        from espetero_amd import abi, device, synth
        self.torch, self.device = torch, device
        self.name, self.bound, self.dtype = name, "hbm", dtype
        self.H, self.Hkv, self.HD, self.bt, self.window = H, H, HD, 0, 0
        self.seqs, self.n_rows, self.tiles, self.n_parts, self.pool_pages = [(0, n_rows)], n_rows, [], 0, 0
        self.dots_only = dots_only
        p, a = synth.make_gate(H, HD, D, dtype, n_rows, seed=seed)
        self.params, self.host = p, a
        tdt = torch.float16 if dtype == abi.ESP_F16 else torch.bfloat16
        dev = lambda x: torch.from_numpy(np.ascontiguousarray(x).view(np.int16)).cuda().view(tdt)  # noqa: E731
        self.n_sets = 4   # rotation sets of X and O so that a step never finds its input in a cache
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        mk = lambda *sh: (torch.randn(*sh, generator=g, device="cuda") * 0.5).to(tdt)  # noqa: E731
        self.X = [dev(a["X"])] + [mk(n_rows, p.x_ld) for _ in range(self.n_sets - 1)]
        self.Os = [dev(a["O"])] + [mk(n_rows, p.q_ld) for _ in range(self.n_sets - 1)]
        self.O = self.Os[0]
        self.Wg = dev(a["Wg"])
        self.dots = torch.zeros(n_rows, H, dtype=torch.float32, device="cuda")
        self.alg_bytes = n_rows * D * 2 + H * D * 2 + (n_rows * H * 4 if dots_only else 2 * n_rows * H * HD * 2)
        self.alg_flops = 0

    def step(self, i):
        k = i % self.n_sets
        self.device.head_gate(self.params, None if self.dots_only else self.Os[k], self.X[k], self.Wg,
                              self.dots if self.dots_only else None, self.n_rows)

    def launch(self, i, l=0):
        self.step(i)


class ChunkedPrefill:
    """One sequence of 8192 tokens in four 2048-token chunks against the paged cache: chunk c's K / V rows are
    appended (esp_kv_save), then it attends to the 2048 c cached tokens and causally to itself, its own rows read
    from the pool (esp_attn_forward without Kb / Vb). A step is the whole sequence: 4 x (append + attention +
    split-K merge). rows_in_pool=False: the attention takes the rows as Kb / Vb (a staging copy of V in front of the
    kernel) and the append follows it."""

    launches_per_step = 4

    def __init__(self, name, H=40, Hkv=8, HD=128, chunk=2048, n_chunks=4, bt=16, seed=3, workgroups=None, rows_in_pool=True):
        self.rows_in_pool = rows_in_pool
        import torch
        from espetero_amd import abi, device, host, synth
        self.torch, self.device = torch, device
        self.name, self.bound, self.dtype = name, "mfma", abi.ESP_BF16
        self.H, self.Hkv, self.HD, self.bt, self.window = H, Hkv, HD, bt, 0
        N = chunk * n_chunks
        self.seqs, self.n_rows = [(0, N)], N
        p = synth.make_params(H, Hkv, HD, self.dtype, bt, rows_per_tile=128)
        p.rows_per_tile = device.plan_hint3(p)[2]
        self.params = p
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        mk = lambda *sh: (torch.randn(*sh, generator=g, device="cuda") * 0.5).to(torch.bfloat16)  # noqa: E731
        self.Q, self.Kb, self.Vb = mk(N, H * HD), mk(N, Hkv * HD), mk(N, Hkv * HD)
        self.O = torch.zeros_like(self.Q)
        n_pages = N // bt
        self.n_sets, self.pool_pages = 2, 2 * n_pages
        self.pool = torch.zeros(self.pool_pages * 2 * bt * Hkv * HD, dtype=torch.bfloat16, device="cuda")
        perm = np.random.default_rng(seed).permutation(self.pool_pages).astype(np.int32)
        resident, groups = device.plan_hint(p)
        opts = host.options_mi355x(p.rows_per_tile, workgroups or resident)
        for k, v in PLAN_TWEAK.items():
            setattr(opts, k, v)
        self.sets, self.tiles, self.n_parts = [], [], 0
        for s_ in range(self.n_sets):
            table = perm[s_ * n_pages:(s_ + 1) * n_pages]
            chunks = []
            for c in range(n_chunks):
                trees = np.array([(0, c * chunk, 0, chunk)], abi.TREE_DT)
                tiles, jobs, n_parts = host.plan_tiles(trees, groups, 0, None, opts)
                dp = device.DevicePass(p, trees, tiles, jobs, n_parts, chunk, table, None, None, pool_blocks=self.pool_pages,
                                       rows_in_pool=rows_in_pool)
                tok = c * chunk + np.arange(chunk)
                e = np.zeros(chunk, abi.KVSAVE_DT)
                e["src_row"], e["block"], e["pos"] = np.arange(chunk), table[tok // bt], tok % bt
                chunks.append((dp, device.to_dev(e), slice(c * chunk, (c + 1) * chunk)))
                if s_ == 0:
                    self.tiles.extend(tiles)
                    self.n_parts += n_parts
            self.sets.append(chunks)
        pairs = sum(chunk * c * chunk + chunk * (chunk + 1) // 2 for c in range(n_chunks))
        self.alg_flops = 4 * HD * H * pairs
        self.alg_bytes = 0

    def launch(self, i, l=0):
        """The attention kernel of chunk l alone (the pool holds the sequence from the steps before)."""
        dp, saves, rows = self.sets[i % self.n_sets][l]
        if self.rows_in_pool:
            dp.run(self.Q[rows], None, None, self.pool, self.O[rows], merge=False)
        else:
            dp.run(self.Q[rows], self.Kb[rows], self.Vb[rows], self.pool, self.O[rows], merge=False)

    def step(self, i):
        d = self.device
        for c, (dp, saves, rows) in enumerate(self.sets[i % self.n_sets]):
            if self.rows_in_pool:
                d.kv_save(self.params, self.Kb[rows], self.Vb[rows], self.pool, saves, rows.stop - rows.start)
                dp.run(self.Q[rows], None, None, self.pool, self.O[rows])
            else:
                dp.run(self.Q[rows], self.Kb[rows], self.Vb[rows], self.pool, self.O[rows])
                d.kv_save(self.params, self.Kb[rows], self.Vb[rows], self.pool, saves, rows.stop - rows.start)


class LayerMix:
    """Six consecutive attention layers of the sliding + global model: five with the 1024-token window,
    one with full attention, as one step (decode or prefill shape)."""

    launches_per_step = 6

    def __init__(self, name, sliding, full):
        self.name, self.sliding, self.full = name, sliding, full
        for k in ("bound", "dtype", "H", "Hkv", "HD", "bt", "seqs", "n_rows", "params", "n_sets", "torch", "device"):
            setattr(self, k, getattr(full, k))
        self.window = sliding.window
        self.tiles = list(sliding.tiles) * 5 + list(full.tiles)
        self.n_parts = 5 * sliding.n_parts + full.n_parts
        self.pool_pages = sliding.pool_pages + full.pool_pages
        self.alg_bytes = 5 * sliding.alg_bytes + full.alg_bytes
        self.alg_flops = 5 * sliding.alg_flops + full.alg_flops
        self.O = full.O

    def step(self, i):
        for l in range(6):
            w = self.full if l == 5 else self.sliding
            w.step(6 * i + l)

    def launch(self, i, l=0):
        (self.full if l == 5 else self.sliding).launch(i)


class DecodeStep:
    """The attention part of one decode step of one layer, from the fp32 fused projection to O: esp_attn_prep (with
    the folded append) followed by esp_attn_forward, or the two as the one call esp_attn_decode_fused."""

    def __init__(self, w, kind, fused, seed=11):
        import torch
        from espetero_amd import device, synth
        self.w, self.fused, self.torch, self.device = w, fused, torch, device
        self.name = w.name + ("_step_fused" if fused else "_step")
        n, bt = w.n_rows, w.bt
        self.pp, a = synth.make_prep(kind, w.H, w.Hkv, w.HD, w.dtype, n, seed=seed, bt=bt)
        dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        self.X = [torch.randn(n, self.pp.x_ld, generator=g, device="cuda") * 1.5 for _ in range(min(4, w.n_sets))]
        self.qn_w, self.kn_w = dev(a["qn_w"]), dev(a["kn_w"])
        self.inv_freq, self.rope_sel, self.pos = dev(a["inv_freq"]), dev(a["rope_sel"]), dev(w.pos)
        # each row's K / V go to entry P of its own sequence, in the blocks of the rotation set the step reads
        self.tables = []
        for blocks in w.tables:
            t = np.full((n, 4), -1, np.int32)
            for tr in w.trees:
                P = int(tr["P"])
                t[int(tr["base"]), :2] = blocks[int(tr["table"]) + P // bt], P % bt
            self.tables.append(dev(t))
        for dp in w.passes:   # the position array serves the prep too: every pass holds it, windowed or not
            dp.pos = self.pos

    def step(self, i):
        w, d = self.w, self.device
        k = i % w.n_sets
        dp, X = w.passes[k], self.X[i % len(self.X)]
        if self.fused:
            d.decode_fused(self.pp, w.params, X, self.qn_w, self.kn_w, self.pos, self.inv_freq, self.rope_sel, self.tables[k], w.pool, dp, w.O)
        else:
            d.attn_prep(self.pp, X, self.qn_w, self.kn_w, self.pos, self.inv_freq, self.rope_sel, w.Q, w.Kb, w.Vb, self.tables[k], w.pool, w.n_rows)
            dp.run(w.Q, w.Kb, w.Vb, w.pool, w.O)


class PrefillStep:
    """The attention part of the chunked prefill of one layer from the fp32 fused projection to O, chunk by chunk:
    esp_attn_prep, esp_attn_forward with the rows as Kb / Vb (a staging copy of V in front of the kernel), esp_kv_save;
    or, folded: esp_attn_prep with the row table and no Kb / Vb of its own, esp_attn_forward reading the rows from the pool."""

    def __init__(self, w, folded, seed=13):
        import torch
        from espetero_amd import device, synth
        self.w, self.folded, self.torch, self.device = w, folded, torch, device
        self.name = w.name + ("_step_folded" if folded else "_step")
        N, bt = w.n_rows, w.bt
        self.pp, a = synth.make_prep("omni", w.H, w.Hkv, w.HD, w.dtype, N, seed=seed, bt=bt, max_pos=1)
        a["pos"][:, :3] = np.arange(N)[:, None]
        dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        self.X = torch.randn(N, self.pp.x_ld, generator=g, device="cuda") * 1.5
        self.qn_w, self.kn_w, self.pos = dev(a["qn_w"]), dev(a["kn_w"]), dev(a["pos"])
        self.inv_freq, self.rope_sel = dev(a["inv_freq"]), dev(a["rope_sel"])
        self.tables = []
        for chunks in w.sets:
            table = chunks[0][0].blocks.cpu().numpy()
            t = np.full((N, 4), -1, np.int32)
            t[:, 0], t[:, 1] = table[np.arange(N) // bt], np.arange(N) % bt
            self.tables.append(dev(t))
        # the same planned passes in both forms: the records do not depend on where the rows are read
        self.passes = [[device.DevicePass(w.params, dp.trees_host, dp.tiles_host, dp.jobs_host, dp.n_parts, dp.n_rows, table_of(chunks), None, None,
                                          rows_in_pool=folded) for dp, _, _ in chunks] for chunks in w.sets]

    def step(self, i):
        w, d = self.w, self.device
        k = i % w.n_sets
        for c, (dp0, saves, rows) in enumerate(w.sets[k]):
            dp = self.passes[k][c]
            n = rows.stop - rows.start
            args = (self.pp, self.X[rows], self.qn_w, self.kn_w, self.pos[rows], self.inv_freq, self.rope_sel, w.Q[rows])
            if self.folded:
                d.attn_prep(*args, None, None, self.tables[k][rows], w.pool, n)
                dp.run(w.Q[rows], None, None, w.pool, w.O[rows])
            else:
                d.attn_prep(*args, w.Kb[rows], w.Vb[rows], None, None, n)
                dp.run(w.Q[rows], w.Kb[rows], w.Vb[rows], w.pool, w.O[rows])
                d.kv_save(w.params, w.Kb[rows], w.Vb[rows], w.pool, saves, n)


def table_of(chunks):
    return chunks[0][0].blocks.cpu().numpy()


def prefill_step_fusion(args, torch, emit=True, steps=10, warmup=2):
    """Step time of the attention part of the chunked prefill (config 3: four chunks) from the fp32 projection to O,
    with the rows handed from the prep to the attention through Kb / Vb and appended afterwards, against the folded form."""
    w = make_workload("c3_chunked_prefill", args.workgroups or None, False, args.page)
    rec, outs, pools = {}, [], []
    for folded in (False, True):
        s = PrefillStep(w, folded)
        w.O.zero_()
        w.pool.zero_()
        s.step(0)
        torch.cuda.synchronize()
        outs.append(w.O.clone())
        pools.append(w.pool.clone())
        for i in range(warmup):
            s.step(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            s.step(i)
        torch.cuda.synchronize()
        tag = "folded" if folded else "three_calls"
        rec[tag + "_eager_us"] = round((time.perf_counter() - t0) / steps * 1e6, 2)
        rec[tag + "_graph_us"] = graph_replay(s, torch, steps=2, replays=4).get("us_per_step")
    rec["identical_output"] = bool(torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16)))
    rec["identical_pool"] = bool(torch.equal(pools[0].view(torch.int16), pools[1].view(torch.int16)))
    parts = 1 if w.n_parts else 0
    rec["dispatches_per_chunk"] = {"three_calls": 4 + parts, "folded": 2 + parts}   # prep, staging copy, attention, [merge,] append | prep, attention[, merge]
    out = {"metric": "chunked prefill attention step, prep + attention (+ append)", "unit": "us", "steps": steps, "config": "c3_chunked_prefill", **rec}
    if emit:
        print(json.dumps(out), flush=True)
    return out


def decode_step_fusion(args, torch, names=("c1_single_decode", "c2_batched_decode", "c4_decode_sliding", "c4_decode_global"), emit=True):
    """Step time of the attention part of a decode layer with and without the prep fused into the attention kernel:
    eager wall time per step and the time per step of 16 steps replayed from one HIP graph."""
    out = {"metric": "decode attention step, prep + attention", "unit": "us", "steps": args.steps, "warmup": args.warmup, "configs": {}}
    for name in names:
        kind = "omni" if name.startswith(("c1", "c2")) else "gemma"
        w = make_workload(name, args.workgroups or None, args.tables == "contiguous", args.page)
        rec = {}
        outs = []
        for fused in (False, True):
            s = DecodeStep(w, kind, fused)
            w.O.zero_()
            s.step(0)
            torch.cuda.synchronize()
            outs.append(w.O.clone())
            for i in range(args.warmup):
                s.step(i)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(args.steps):
                s.step(i)
            torch.cuda.synchronize()
            tag = "fused" if fused else "two_calls"
            rec[tag + "_eager_us"] = round((time.perf_counter() - t0) / args.steps * 1e6, 2)
            rec[tag + "_graph_us"] = graph_replay(s, torch).get("us_per_step")
        rec["identical_output"] = bool(torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16)))
        rec["dispatches"] = {"two_calls": 2 + (1 if w.n_parts else 0), "fused": 1 + (1 if w.n_parts else 0)}
        out["configs"][name] = rec
        del w
        torch.cuda.empty_cache()
    if emit:
        print(json.dumps(out), flush=True)
    return out


def make_workload(name, workgroups=None, contiguous=False, page=16):
    from espetero_amd import abi, synth
    from functools import partial
    F16, BF16 = abi.ESP_F16, abi.ESP_BF16
    Workload_ = partial(Workload, workgroups=workgroups, contiguous=contiguous)
    if name in ("c4_decode_mix", "c4_prefill_mix"):   # the 5 : 1 layer mix of config 4 as one step
        kind = name[3:-4]
        return LayerMix(name, make_workload(f"c4_{kind}_sliding", workgroups, contiguous, page),
                        make_workload(f"c4_{kind}_global", workgroups, contiguous, page))
    if name in ("c3_chunked_prefill", "c3_chunked_prefill_kb"):   # the whole of config 3 as one step; _kb: rows handed over as Kb / Vb
        return ChunkedPrefill(name, bt=page, workgroups=workgroups, rows_in_pool=not name.endswith("_kb"))
    if name == "c3_attn_prep":   # the rows of one C3 prefill chunk, Qwen3-Omni arrangement (82_qwen3_omni.metal:30-88)
        return PrepWorkload(name, "omni", 40, 8, 128, BF16, 2048, bt=page)
    if name == "c4_attn_prep":   # the rows of one C4 prefill pass, Qwen3.5 arrangement (40_attention.metal:9-102)
        return PrepWorkload(name, "qwen35", 16, 8, 256, F16, 8 * 1024, bt=page)
    if name in ("c4_head_gate", "c4_head_gate_dots"):   # the rows of one C4 prefill pass; model width 2560 (assumed: a 4B Spark)
        return GateWorkload(name, 16, 256, 2560, F16, 8 * 1024, dots_only=name.endswith("dots"))
    if name == "c1_single_decode":
        return Workload_(name, 32, 4, 128, F16, page, [(1024, 1)], pool_pages=(64 * 16) * 16 // page, seed=1)
    if name == "c2_batched_decode":
        lens = synth.c2_lengths()
        return Workload_(name, 32, 4, 128, F16, page, [(L, 1) for L in lens], pool_pages=(65536) * 16 // page, seed=2)
    if name.startswith("c2_equal_"):   # config 2's geometry with 16 sequences of one length: what a decode pass costs beside its bytes
        L = int(name[len("c2_equal_"):])
        return Workload_(name, 32, 4, 128, F16, page, [(L, 1)] * 16, pool_pages=(65536) * 16 // page, seed=2)
    if name == "c4_decode_sliding":
        return Workload_(name, 16, 8, 256, F16, page, [(16384, 1)] * 8, window=1024, pool_pages=(8 * 1025 * 4) * 16 // page, seed=4)
    if name == "c4_decode_global":
        return Workload_(name, 16, 8, 256, F16, page, [(16384, 1)] * 8, pool_pages=(8 * 1025 * 4) * 16 // page, seed=4)
    if name == "c5_verify":
        return Workload_(name, 32, 4, 128, F16, page, [(32768, 4)] * 8, rows_per_tile=4,
                        desc_fn=lambda M: synth.verify_desc(M, 1), pool_pages=(65536 + 64) * 16 // page, seed=5)
    # Gemma 4's full-attention layers as the reference runs them (head dim 512, 16 query heads on 2 KV heads:
    # gemma.h:125-150), on config 4's sequences: what config 4's "global" layers are in the real model.
    if name == "g4_global512_decode":
        return Workload_(name, 16, 2, 512, F16, page, [(16384, 1)] * 8, pool_pages=(8 * 1025 * 4) * 16 // page, seed=6)
    if name in ("g4_global512_verify", "g4_global512_verify_2row_tiles"):   # 4-row verify trees there: 32 packed rows in one pass over K / V, or as two 2-row tiles
        return Workload_(name, 16, 2, 512, F16, page, [(16384, 4)] * 8, rows_per_tile=4 if name.endswith("verify") else 2,
                        desc_fn=lambda M: synth.verify_desc(M, 1), pool_pages=(8 * 1025 * 4) * 16 // page, seed=6)
    if name == "g4_global512_prefill":
        return Workload_(name, 16, 2, 512, F16, page, [(15360, 1024)] * 8, rows_per_tile=128, pool_pages=(8 * 1024 * 2) * 16 // page,
                        seed=6, bound="mfma")
    if name.startswith("c3_prefill_p"):
        P = int(name[len("c3_prefill_p"):])
        return Workload_(name, 40, 8, 128, BF16, page, [(P, 2048)], rows_per_tile=128, pool_pages=(1024) * 16 // page, seed=3, bound="mfma")
    if name == "c4_prefill_sliding":
        return Workload_(name, 16, 8, 256, F16, page, [(15360, 1024)] * 8, window=1024, rows_per_tile=128,
                        pool_pages=(8 * 1024 * 2) * 16 // page, seed=4, bound="mfma")
    if name == "c4_prefill_sliding_chunk2048":   # config 4's sliding layer with the reference's own chunk (2048 rows): twice the window
        return Workload_(name, 16, 8, 256, F16, page, [(14336, 2048)] * 4, window=1024, rows_per_tile=128,
                        pool_pages=(8 * 1024 * 2) * 16 // page, seed=4, bound="mfma")
    if name == "c4_prefill_sliding_window512":   # ... and with a window half the chunk
        return Workload_(name, 16, 8, 256, F16, page, [(15360, 1024)] * 8, window=512, rows_per_tile=128,
                        pool_pages=(8 * 1024 * 2) * 16 // page, seed=4, bound="mfma")
    if name == "one_prompt_first_chunk":   # config 4's global layer on one prompt's first 2048 rows: 16 tiles x 16 heads, one per compute unit
        return Workload_(name, 16, 8, 256, F16, page, [(0, 2048)], rows_per_tile=128, pool_pages=4096 * 16 // page, seed=4, bound="mfma")
    if name == "one_prompt_first_chunk_hd128":   # the same rows on 16 heads of 128 dims: half of the slots of the narrower kernel
        return Workload_(name, 16, 8, 128, BF16, page, [(0, 2048)], rows_per_tile=128, pool_pages=4096 * 16 // page, seed=4, bound="mfma")
    if name == "c4_prefill_global":
        return Workload_(name, 16, 8, 256, F16, page, [(15360, 1024)] * 8, rows_per_tile=128, pool_pages=(8 * 1024 * 2) * 16 // page, seed=4,
                        bound="mfma")
    raise SystemExit(f"unknown workload {name}")


def measured_traffic(workload):
    """HBM bytes one launch of the dominant kernel moves, as measured with the rocprofv3 FETCH_SIZE and
    WRITE_SIZE counters (each scaled by what the same counter reads for a plain 256 MiB copy); the
    summaries under profiles/ show the runs. A step of several launches (the chunked prefill, the layer mixes) is
    the sum over its launches. None for a workload that has not been measured."""
    chunks = ["c3_prefill_p0", "c3_prefill_p2048", "c3_prefill_p4096", "c3_prefill_p6144"]   # one launch per chunk
    parts = {"c3_chunked_prefill": chunks, "c3_chunked_prefill_kb": chunks,
             "c4_decode_mix": ["c4_decode_sliding"] * 5 + ["c4_decode_global"],
             "c4_prefill_mix": ["c4_prefill_sliding"] * 5 + ["c4_prefill_global"]}.get(workload, [workload])
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            t = json.load(f)
        return sum(int(t[x]["hbm_bytes_per_launch"]) for x in parts)
    except (OSError, KeyError, ValueError):
        return None


def traffic_source():
    """Where roofline.traffic comes from: the commit the rocprofv3 counter runs under profiles/ were last taken at,
    and the commit of each workload's own runs."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            t = json.load(f)
        per = {k: v.get("measured_at_commit") for k, v in t.items() if isinstance(v, dict) and "measured_at_commit" in v}
        return {"file": "profiles/traffic.json", "measured_at_commit": t.get("_measured_at_commit"),
                "per_workload": per, "note": t.get("_note")}
    except (OSError, ValueError):
        return None


PLAN_TWEAK = {}   # fields of the planner's options set from the command line


WORKLOADS = ["c1_single_decode", "c2_batched_decode", "c3_prefill_p0", "c3_prefill_p2048", "c3_prefill_p4096",
             "c3_prefill_p6144", "c4_decode_sliding", "c4_decode_global", "c4_prefill_sliding", "c4_prefill_global",
             "c5_verify", "c4_decode_mix", "c4_prefill_mix", "c3_chunked_prefill", "c3_chunked_prefill_kb", "c3_attn_prep", "c4_attn_prep",
             "c4_head_gate", "c4_head_gate_dots", "g4_global512_decode", "g4_global512_verify", "g4_global512_verify_2row_tiles",
             "g4_global512_prefill", "one_prompt_first_chunk", "one_prompt_first_chunk_hd128", "c4_prefill_sliding_chunk2048",
             "c4_prefill_sliding_window512"]


def cpu_baseline(w, budget_s=20.0):
    """The CPU checker (scalar C restatement of the reference semantics) on a bounded sample of
    the same workload: whole sequences, gathered from the device pool through esp_kv_gather into a
    reference-layout pool. Timed single-threaded; the all-core time is reported beside it."""
    import torch
    from espetero_amd import abi, device, synth
    from oracle import binding as ob
    p = w.params
    kvw = p.Hkv * p.head_dim
    # ~1 GFLOP/s scalar with storage conversions: size the sample to the budget
    flops_budget = 1.0e9 * budget_s
    seqs, tot = [], 0.0
    for i, (P, M) in enumerate(w.seqs):
        rows = min(M, max(1, int(flops_budget // max(1.0, 4.0 * p.head_dim * p.H * (P + M)))))
        f = 4.0 * p.head_dim * p.H * rows * (P + rows)
        if seqs and tot + f > flops_budget:
            break
        seqs.append((i, P, rows))
        tot += f
    bt = p.bt
    n_blocks = sum((P + bt - 1) // bt for _, P, _ in seqs) + 1
    pool_ref = np.zeros(n_blocks * 2 * bt * kvw, np.uint16)
    pv = pool_ref.reshape(n_blocks, 2, bt, kvw)
    trees = np.zeros(len(seqs), abi.TREE_DT)
    table, nb_used, base = [], 0, 0
    table_dev = w.passes[0].blocks
    rows_total = sum(r for _, _, r in seqs)
    Q = np.zeros((rows_total, p.q_ld), np.uint16)
    Kb = np.zeros((rows_total, p.kv_ld), np.uint16)
    Vb = np.zeros((rows_total, p.kv_ld), np.uint16)
    desc = np.zeros((rows_total, 4), np.int32)
    pos = np.zeros((rows_total, 4), np.int32)
    for (i, P, rows) in seqs:
        t = w.trees[i]
        nb = (P + bt - 1) // bt
        if P:
            K = torch.zeros(P * kvw, dtype=torch.int16, device="cuda")
            V = torch.zeros_like(K)
            device.kv_gather(p, w.pool, table_dev[int(t["table"]):], P, K, V)
            torch.cuda.synchronize()
            Kh = np.zeros((nb * bt, kvw), np.uint16)
            Vh = np.zeros((nb * bt, kvw), np.uint16)
            Kh[:P] = K.cpu().numpy().view(np.uint16).reshape(P, kvw)
            Vh[:P] = V.cpu().numpy().view(np.uint16).reshape(P, kvw)
            pv[nb_used:nb_used + nb, 0] = Kh.reshape(nb, bt, kvw)
            pv[nb_used:nb_used + nb, 1] = Vh.reshape(nb, bt, kvw)
        idx = [k for k, s in enumerate(seqs) if s[0] == i][0]
        trees[idx] = (base, P, len(table), rows)
        table.extend(range(nb_used, nb_used + nb))
        nb_used += nb
        b0 = int(t["base"])
        Q[base:base + rows] = w.Q[b0:b0 + rows].view(torch.int16).cpu().numpy().view(np.uint16)
        Kb[base:base + rows] = w.Kb[b0:b0 + rows].view(torch.int16).cpu().numpy().view(np.uint16)
        Vb[base:base + rows] = w.Vb[b0:b0 + rows].view(torch.int16).cpu().numpy().view(np.uint16)
        desc[base:base + rows] = w.desc[b0:b0 + rows]
        pos[base:base + rows] = w.pos[b0:b0 + rows]
        base += rows
    blocks = np.asarray(table if table else [0], np.int32)
    pr = synth.make_params(p.H, p.Hkv, p.head_dim, p.dtype, bt, window=p.window, rows_per_tile=p.rows_per_tile)
    # work of the sample, counted as for the GPU
    vis_keys, pairs = 0, 0
    for _, P, rows in seqs:
        for r in range(rows):
            lo = max(0, P + r - p.window + 1) if p.window > 0 else 0
            pairs += (P + r + 1) - lo
        lo = max(0, P - p.window + 1) if p.window > 0 else 0
        vis_keys += (P + rows) - lo
    s_bytes = vis_keys * kvw * 2 * 2 + 2 * rows_total * p.H * p.head_dim * 2 + ((vis_keys + bt - 1) // bt) * 4
    s_flops = 4 * p.head_dim * p.H * pairs
    t0 = time.perf_counter()
    o1 = ob.attn_direct(pr, Q, Kb, Vb, pool_ref, blocks, desc, pos, trees, n_threads=1)
    t1 = time.perf_counter() - t0
    ncores = min(16, os.cpu_count() or 1)
    t0 = time.perf_counter()
    ob.attn_direct(pr, Q, Kb, Vb, pool_ref, blocks, desc, pos, trees, n_threads=ncores)
    tn = time.perf_counter() - t0
    # the sample doubles as a parity spot check of the benchmarked device path
    max_err = None
    if all(rows == M for (_, _, rows), (_, M) in zip(seqs, [w.seqs[i] for i, _, _ in seqs])):
        got = w.O.view(torch.int16).cpu().numpy().view(np.uint16)
        errs = []
        base = 0
        for (i, P, rows) in seqs:
            b0 = int(w.trees[i]["base"])
            errs.append(ob.beyond_rounding(ob.to_f32(got[b0:b0 + rows], p.dtype), ob.to_f32(o1[base:base + rows], p.dtype), p.dtype, True))
            base += rows
        max_err = float(max(errs))
    unit = "GB/s" if w.bound == "hbm" else "TFLOP/s"
    val1 = s_bytes / t1 / 1e9 if w.bound == "hbm" else s_flops / t1 / 1e12
    valn = s_bytes / tn / 1e9 if w.bound == "hbm" else s_flops / tn / 1e12
    whole = w.alg_bytes if w.bound == "hbm" else w.alg_flops
    return {"value": round(val1, 6), "unit": unit, "cores": 1, "kind": "port",
            "sample": f"{len(seqs)} of {len(w.seqs)} sequences ({rows_total} of {w.n_rows} rows, {vis_keys} visible keys), "
                      f"{t1:.2f} s single-threaded",
            "extrapolation_factor": round(whole / max(s_bytes if w.bound == "hbm" else s_flops, 1), 3),
            "all_cores": {"value": round(valn, 6), "cores": ncores, "seconds": round(tn, 3)},
            "host_cpus": os.cpu_count(), "max_abs_err_vs_gpu": max_err}


def prep_cpu_baseline(w):
    """The CPU checker's attn_prep on the workload's own rows (rotation set 0), single-threaded."""
    from oracle import binding as ob
    a, p = w.host, w.params
    rows = min(w.n_rows, 2048)
    t0 = time.perf_counter()
    Q, K, V = ob.attn_prep(p, a["X"][:rows], a["qn_w"], a["kn_w"], a["pos"][:rows], a["inv_freq"], a["rope_sel"], rows)
    dt = time.perf_counter() - t0
    bits = lambda t: t.view(w.torch.int16).cpu().numpy().view(np.uint16)  # noqa: E731
    f = lambda b: ob.to_f32(b, p.dtype).astype(np.float64)  # noqa: E731
    err = max(float(np.abs(f(bits(g)[:rows]) - f(c)).max()) for g, c in ((w.Q, Q), (w.Kb, K), (w.Vb, V)))
    return {"value": round(w.alg_bytes * rows / w.n_rows / dt / 1e9, 6), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{rows} of {w.n_rows} rows, {dt:.2f} s single-threaded", "host_cpus": os.cpu_count(),
            "max_abs_err_vs_gpu": err}


def gate_cpu_baseline(w):
    """The CPU checker's head gate on rows of rotation set 0, single-threaded, against a fresh GPU run on the same rows."""
    import torch
    from oracle import binding as ob
    a, p = w.host, w.params
    rows = min(w.n_rows, 1024)
    t0 = time.perf_counter()
    want, want_dots = ob.head_gate(p, a["O"][:rows], a["X"][:rows], a["Wg"], rows, want_dots=True)
    dt = time.perf_counter() - t0
    O = torch.from_numpy(np.ascontiguousarray(a["O"][:rows]).view(np.int16)).cuda()
    w.device.head_gate(p, O, w.X[0], w.Wg, w.dots, rows)
    torch.cuda.synchronize()
    f = lambda b: ob.to_f32(b, p.dtype).astype(np.float64)  # noqa: E731
    err = float(np.abs(f(O.cpu().numpy().view(np.uint16)) - f(want)).max())
    derr = float(np.abs(w.dots[:rows].cpu().numpy() - want_dots).max())
    return {"value": round(w.alg_bytes * rows / w.n_rows / dt / 1e9, 6), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{rows} of {w.n_rows} rows, {dt:.2f} s single-threaded", "host_cpus": os.cpu_count(),
            "max_abs_err_vs_gpu": err, "max_abs_dot_err_vs_gpu": derr}


def chunked_cpu_baseline(w, rows=24):
    """The CPU checker on the last `rows` rows of the sequence (the longest rows: every earlier token cached),
    gathered from the pool the last step filled."""
    import torch
    from espetero_amd import abi, device
    from oracle import binding as ob
    p = w.params
    N, kvw, bt = w.n_rows, p.Hkv * p.head_dim, p.bt
    P = N - rows
    chunks = w.sets[0]
    table = chunks[0][0].blocks
    K = torch.zeros(P * kvw, dtype=torch.int16, device="cuda")
    V = torch.zeros_like(K)
    device.kv_gather(p, w.pool, table, P, K, V)
    torch.cuda.synchronize()
    nb = (P + bt - 1) // bt
    pool_ref = np.zeros((nb + 1) * 2 * bt * kvw, np.uint16)
    pv = pool_ref.reshape(nb + 1, 2, bt, kvw)
    Kh, Vh = np.zeros((nb * bt, kvw), np.uint16), np.zeros((nb * bt, kvw), np.uint16)
    Kh[:P] = K.cpu().numpy().view(np.uint16).reshape(P, kvw)
    Vh[:P] = V.cpu().numpy().view(np.uint16).reshape(P, kvw)
    pv[:nb, 0], pv[:nb, 1] = Kh.reshape(nb, bt, kvw), Vh.reshape(nb, bt, kvw)
    bits = lambda t: t.view(torch.int16).cpu().numpy().view(np.uint16)  # noqa: E731
    Q, Kb, Vb = bits(w.Q[P:]), bits(w.Kb[P:]), bits(w.Vb[P:])
    trees = np.array([(0, P, 0, rows)], abi.TREE_DT)
    z = np.zeros((rows, 4), np.int32)
    t0 = time.perf_counter()
    O = ob.attn_direct(p, Q, Kb, Vb, pool_ref, np.arange(nb, dtype=np.int32), z, z, trees, n_threads=1)
    dt = time.perf_counter() - t0
    flops = 4 * p.head_dim * p.H * sum(P + r + 1 for r in range(rows))
    err = ob.beyond_rounding(ob.to_f32(bits(w.O[P:]), p.dtype), ob.to_f32(O, p.dtype), p.dtype, True)
    return {"value": round(flops / dt / 1e12, 9), "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"the last {rows} of {N} rows ({flops / 1e9:.2f} GFLOP), {dt:.2f} s single-threaded",
            "extrapolation_factor": round(w.alg_flops / flops, 3),
            "host_cpus": os.cpu_count(), "max_abs_err_vs_gpu": err}


def graph_replay(w, torch, steps=16, replays=8):
    """The same steps captured once in a HIP graph and replayed: what a caller that enqueues a chain of
    passes without host work in between (a decode chain) pays per step."""
    try:
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                for i in range(steps):
                    w.step(i)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(replays):
            g.replay()
        torch.cuda.synchronize()
        return {"us_per_step": round((time.perf_counter() - t0) / (replays * steps) * 1e6, 3), "steps_per_graph": steps}
    except RuntimeError as e:  # reported, never hidden: the timed figures above do not depend on it
        return {"error": str(e).splitlines()[0][:200]}


def spot_check(w, rows=4, threads=8):
    """Parity of what the timed steps left in O, on a sample: the last `rows` rows of the workload's first and
    last sequence (whole trees when they carry a verify descriptor), against the CPU checker. The rows before
    them in the same pass count as cached keys, which the attention's semantics make equivalent
    (kernels/40_attention.metal:245-249: a batch key and the same key in the cache score alike). Returns
    (max abs error, rows checked)."""
    import torch
    from espetero_amd import abi, device, synth
    from oracle import binding as ob
    p = w.params
    kvw, bt = p.Hkv * p.head_dim, p.bt
    bits = lambda t: t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)  # noqa: E731
    w.step(0)   # rotation set 0's block tables are the ones gathered below
    torch.cuda.synchronize()
    worst, checked = 0.0, 0
    plain = not np.any(w.desc)
    for i in sorted({0, len(w.seqs) - 1}):
        P, M = w.seqs[i]
        t = w.trees[i]
        b0 = int(t["base"])
        r = min(rows, M) if plain else M
        Pc = P + M - r                       # cached keys as the sampled rows see them
        nb = (Pc + bt - 1) // bt
        pool_ref = np.zeros((nb + 1) * 2 * bt * kvw, np.uint16)
        pv = pool_ref.reshape(nb + 1, 2, bt, kvw)
        Kh, Vh = np.zeros((nb * bt, kvw), np.uint16), np.zeros((nb * bt, kvw), np.uint16)
        if P:
            K = torch.zeros(P * kvw, dtype=torch.int16, device="cuda")
            V = torch.zeros_like(K)
            device.kv_gather(p, w.pool, w.passes[0].blocks[int(t["table"]):], P, K, V)
            torch.cuda.synchronize()
            Kh[:P], Vh[:P] = bits(K).reshape(P, kvw), bits(V).reshape(P, kvw)
        if M > r:
            Kh[P:Pc] = bits(w.Kb[b0:b0 + M - r])[:, :kvw]
            Vh[P:Pc] = bits(w.Vb[b0:b0 + M - r])[:, :kvw]
        if nb:
            pv[:nb, 0], pv[:nb, 1] = Kh.reshape(nb, bt, kvw), Vh.reshape(nb, bt, kvw)
        sl = slice(b0 + M - r, b0 + M)
        pos = np.zeros((r, 4), np.int32)
        pos[:, :3] = (Pc + np.arange(r))[:, None]
        desc = np.zeros((r, 4), np.int32) if plain else w.desc[sl]
        pr = synth.make_params(p.H, p.Hkv, p.head_dim, p.dtype, bt, window=p.window, rows_per_tile=p.rows_per_tile)
        want = ob.attn_direct(pr, bits(w.Q[sl]), bits(w.Kb[sl]), bits(w.Vb[sl]), pool_ref, np.arange(max(nb, 1), dtype=np.int32),
                              desc, pos, np.array([(0, Pc, 0, r)], abi.TREE_DT), n_threads=threads)
        got = bits(w.O[sl])
        worst = max(worst, ob.beyond_rounding(ob.to_f32(got, p.dtype), ob.to_f32(want, p.dtype), p.dtype, True))
        checked += r
    return worst, checked


def tolerance(dtype=None):
    """The one bar of the path for both element types: max-abs 2e-3 on what is left of a difference once the
    rounding of the stored output itself is taken off (oracle.binding.beyond_rounding)."""
    return 2e-3


_SPIN = {}


def spin(torch, ms):
    """Keeps the GPU busy for about `ms` milliseconds (torch's own bounded spin kernel), so that what is
    enqueued behind it is already in the queue when the GPU gets to it."""
    if "per_ms" not in _SPIN:
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda._sleep(1000000)
        a.record()
        torch.cuda._sleep(4000000)
        b.record()
        torch.cuda.synchronize()
        _SPIN["per_ms"] = 4000000 / max(a.elapsed_time(b), 1e-3)
    torch.cuda._sleep(int(_SPIN["per_ms"] * ms))


def kernel_times(w, torch, n, first_step=0, step_seconds=0.0, reps=5):
    """Durations of the dominant kernel's launches, in milliseconds [reps][launches per step]: for every launch of
    a step, `reps` runs of that launch alone (w.launch: the attention without the merge behind it) repeated back to
    back, timed by two events around the run and divided by the count. Consecutive launches of one stream follow
    each other without a gap (the trace shows the next dispatch beginning where the last one ends), so the quotient
    is the dispatch's own begin-to-end time, and nothing is inserted between the launches that could perturb them:
    an event pair handed to every launch (hipExtLaunchKernelGGL) puts a marker in front of each dispatch, which the
    trace shows costs the stream 9 to 14 us per launch and makes the kernel itself read 2 to 6 % longer. Runs of
    short launches are enqueued behind a few milliseconds of spinning, so that the queue never runs dry."""
    nev = getattr(w, "launches_per_step", 1)
    per = max(step_seconds / nev, 2e-6)
    count = int(min(200, max(8, round(3e-3 / per))))   # launches per run: about 3 ms
    out = np.zeros((reps, nev))
    for l in range(nev):
        for r in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            if per < 2e-4:
                spin(torch, 1.0 + 0.02 * count)
            a.record()
            for i in range(count):
                w.launch(first_step + r * count + i, l)
            b.record()
            torch.cuda.synchronize()
            out[r, l] = a.elapsed_time(b) / count
    return out


def timed_run(w, torch, steps, warmup, kernel_samples=None):
    """30 ms of the workload's own steps to wake the device, `warmup` untimed steps, then exactly `steps` timed ones
    between two device synchronisations with nothing but the steps in the loop: wall seconds per step. The dominant kernel's own durations are taken afterwards, in a
    loop of their own (kernel_times), so that the instrumentation is not part of what the wall clock sees.
    Returns (wall seconds per step, kernel milliseconds [samples][launches per step])."""
    # A GPU that has sat idle while the host built the workload takes milliseconds to leave its low-power state,
    # longer than a handful of 30 us warm-up steps last: keep it busy with the workload's own steps for 30 ms first.
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < (0.03 if w.bound == "hbm" else 0.1):   # matrix-bound passes also settle at the clock their power allows
        w.step(i)
        i += 1
        if i % 64 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    for i in range(warmup):
        w.step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        w.step(warmup + i)
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    return wall, kernel_times(w, torch, steps, warmup + steps, wall)


def kernel_name(w):
    return getattr(w, "kernel", None) or ("attn_stream_kernel" if w.params.rows_per_tile * (w.H // w.Hkv) <= 32
                                          else "attn_tiled512_kernel" if w.HD == 512 else "attn_tiled_kernel")


def roofline(w, per_step_ms):
    """achieved = algorithmic bytes (flops) of the pass / the dominant kernel's mean duration per step."""
    mean, med, mn = float(np.mean(per_step_ms)), float(np.median(per_step_ms)), float(np.min(per_step_ms))
    if w.bound == "hbm":
        work, peak, unit, scale = w.alg_bytes, HBM_PEAK_GBS, "GB/s", 1e9
    else:
        work, peak, unit, scale = w.alg_flops, MFMA_PEAK_TFLOPS, "TFLOP/s", 1e12
    achieved = work / (mean * 1e-3) / scale
    r = {"bound": w.bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit, "frac": round(achieved / peak, 4),
         "traffic": measured_traffic(w.name), "kernel": kernel_name(w), "kernel_us_avg": round(mean * 1e3, 3),
         "kernel_us_median": round(med * 1e3, 3), "kernel_us_min": round(mn * 1e3, 3), "samples": int(len(per_step_ms)),
         "alg_bytes": int(w.alg_bytes), "alg_flops": int(w.alg_flops)}
    return r


def headline(w, wall, per_launch, steps, warmup):
    from espetero_amd import abi
    per_step = per_launch.sum(axis=1)
    if w.bound == "hbm":
        metric = ("attn-prep HBM GB/s" if isinstance(w, PrepWorkload) else
                  "head-gate HBM GB/s" if isinstance(w, GateWorkload) else "decode-attn HBM GB/s")
        unit, value = "GB/s", w.alg_bytes / wall / 1e9
    else:
        metric, unit, value = "prefill-attn TFLOPS", "TFLOP/s", w.alg_flops / wall / 1e12
    return {
        "metric": metric, "value": round(value, 3), "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(wall * 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if w.dtype == abi.ESP_F16 else "bf16", "data": "synthetic",
        "config": {"workload": w.name, "sequences": len(w.seqs), "rows": w.n_rows, "H": w.H, "Hkv": w.Hkv,
                   "head_dim": w.HD, "page": w.bt, "window": w.window, "context_tokens": int(sum(P for P, _ in w.seqs)),
                   "tiles": int(len(w.tiles)), "parts": int(w.n_parts), "rotation_sets": w.n_sets,
                   "pool_pages": w.pool_pages},
        "roofline": roofline(w, per_step),
    }


def cpu_leg(w, torch, budget_s=20.0):
    w.step(0)   # leave rotation set 0's output in O: the CPU sample is checked against it
    torch.cuda.synchronize()
    if isinstance(w, PrepWorkload):
        return prep_cpu_baseline(w)
    if isinstance(w, GateWorkload):
        return gate_cpu_baseline(w)
    if isinstance(w, ChunkedPrefill):
        return chunked_cpu_baseline(w)
    if isinstance(w, LayerMix):
        return mix_cpu_baseline(w, budget_s)
    return cpu_baseline(w, budget_s)


def mix_cpu_baseline(w, budget_s):
    """The 5 : 1 layer mix on the CPU: a sample of each layer kind, each extrapolated to its whole layer, five
    sliding layers and the full one added up as the GPU step adds them."""
    w.full.step(0)      # rotation set 0 of each layer kind: the tables the samples are gathered through
    w.sliding.step(0)
    w.torch.cuda.synchronize()
    g = cpu_baseline(w.full, budget_s * 0.7)
    sl = cpu_baseline(w.sliding, budget_s * 0.3)
    hb = w.bound == "hbm"
    work = lambda x: x.alg_bytes / 1e9 if hb else x.alg_flops / 1e12  # noqa: E731
    secs = 5 * work(w.sliding) / sl["value"] + work(w.full) / g["value"]
    secs_all = 5 * work(w.sliding) / sl["all_cores"]["value"] + work(w.full) / g["all_cores"]["value"]
    errs = [x["max_abs_err_vs_gpu"] for x in (g, sl) if x["max_abs_err_vs_gpu"] is not None]
    return {"value": round((5 * work(w.sliding) + work(w.full)) / secs, 6), "unit": g["unit"], "cores": 1, "kind": "port",
            "sample": "full layer: " + g["sample"] + "; sliding layer: " + sl["sample"],
            "extrapolation_factor": {"full": g["extrapolation_factor"], "sliding": sl["extrapolation_factor"]},
            "all_cores": {"value": round((5 * work(w.sliding) + work(w.full)) / secs_all, 6), "cores": g["all_cores"]["cores"]},
            "host_cpus": os.cpu_count(), "max_abs_err_vs_gpu": max(errs) if errs else None}


def compact(w, torch, steps, warmup):
    """One short record of a benchmark configuration: step time, the dominant kernel's duration and roofline
    fraction, and a parity spot check of the output the timed steps left behind."""
    from espetero_amd import abi
    wall, per_launch = timed_run(w, torch, steps, warmup)
    per_step = per_launch.sum(axis=1)
    r = roofline(w, per_step)
    rec = {"workload": w.name, "bound": w.bound, "steps": steps, "ms_per_step": round(wall * 1e3, 6),
           "value": round((w.alg_bytes / 1e9 if w.bound == "hbm" else w.alg_flops / 1e12) / wall, 3), "unit": r["unit"],
           "kernel": r["kernel"], "kernel_us_median": r["kernel_us_median"], "kernel_us_min": r["kernel_us_min"],
           "kernel_us_avg": r["kernel_us_avg"], "achieved": r["achieved"], "frac": r["frac"],
           "dtype": "f16" if w.dtype == abi.ESP_F16 else "bf16", "tolerance": tolerance(w.dtype)}
    return rec, per_launch


def part_record(name, work, unit_scale, peak, ms):
    """A launch of a multi-launch step on its own (a chunk of the chunked prefill, a layer kind of the mix)."""
    mean = float(np.mean(ms))
    ach = work / (mean * 1e-3) / unit_scale
    return {"part": name, "kernel_us_median": round(float(np.median(ms)) * 1e3, 3), "kernel_us_min": round(float(np.min(ms)) * 1e3, 3),
            "kernel_us_avg": round(mean * 1e3, 3), "achieved": round(ach, 3), "frac": round(ach / peak, 4)}


class Ceilings:
    """The machine's own ceilings, measured in this run by libespetero_ceilings.so: a plain non-temporal
    16-byte-per-lane read of scattered 8 KB pages (and of the same bytes in address order), and the matrix cores
    under a wavefront that issues the prefill kernel's share of vector arithmetic beside them."""

    def __init__(self):
        import ctypes as C
        import torch
        self.torch, self.C = torch, C
        path = os.path.join(ROOT, "espetero_amd", "csrc", "libespetero_ceilings.so")
        if not os.path.exists(path):
            raise SystemExit(f"{path} is not built (run __graft_entry__.build())")
        self.lib = C.CDLL(path)
        V, I = C.c_void_p, C.c_int32
        self.lib.esp_ceiling_hbm_read.argtypes = [V, V, I, I, I, I, V, V, V, V]
        self.lib.esp_ceiling_mfma_issue.argtypes = [I, I, I, I, I, V, V, V, V]
        self.lib.esp_ceiling_prefill_step.argtypes = [I, I, I, I, I, V, V, V, V, V, V]
        self.lib.esp_ceiling_prefill_step256.argtypes = [I, I, I, I, V, V, V, V, V, V]

    def _events(self, n):
        t = self.torch
        evs = [(t.cuda.Event(enable_timing=True), t.cuda.Event(enable_timing=True)) for _ in range(n)]
        for a, b in evs:
            a.record()
            b.record()
        t.cuda.synchronize()
        return evs

    def hbm_read(self, mbytes=(141, 537, 1074), page_bytes=8192, reps=12, workgroups=2 * N_CU):
        """GB/s of the plain read at each size: scattered pages (a seeded permutation of a 4 GiB buffer) and
        address order, non-temporal and ordinary loads. Each repetition reads other pages than the one before."""
        t = self.torch
        total = 4 << 30
        buf = t.empty(total, dtype=t.uint8, device="cuda")
        buf.fill_(1)
        sink = t.zeros(4, dtype=t.int32, device="cuda")
        n_all = total // page_bytes
        perm = t.from_numpy(np.random.default_rng(11).permutation(n_all).astype(np.int32)).cuda()
        st = self.C.c_void_p(t.cuda.current_stream().cuda_stream)
        out = []
        for mb in mbytes:
            n_pages = mb * 1000000 // page_bytes
            rec = {"bytes": n_pages * page_bytes, "page_bytes": page_bytes, "workgroups": workgroups}
            for label, scattered, nt in (("scattered_nt", True, 1), ("scattered", True, 0), ("contiguous_nt", False, 1)):
                evs = self._events(reps)
                for k, (a, b) in enumerate(evs):
                    off = (k * n_pages) % (n_all - n_pages)
                    pages = self.C.c_void_p(perm.data_ptr() + 4 * off) if scattered else None
                    base = self.C.c_void_p(buf.data_ptr() + (0 if scattered else off * page_bytes))
                    rc = self.lib.esp_ceiling_hbm_read(base, pages, n_pages, page_bytes, nt, workgroups,
                                                       self.C.c_void_p(sink.data_ptr()), st, self.C.c_void_p(a.cuda_event),
                                                       self.C.c_void_p(b.cuda_event))
                    assert rc == 0, rc
                t.cuda.synchronize()
                ms = np.array([a.elapsed_time(b) for a, b in evs][2:])
                rec[label] = {"GBs_median": round(rec["bytes"] / float(np.median(ms)) / 1e6, 1),
                              "GBs_best": round(rec["bytes"] / float(ms.min()) / 1e6, 1), "us_median": round(float(np.median(ms)) * 1e3, 2)}
            out.append(rec)
        del buf, perm
        t.cuda.empty_cache()
        return out

    def mfma_issue(self, mixes=((0, 0, 1), (0, 0, 0), (2, 1, 1), (4, 1, 1), (4, 1, 0)), iters=2000, workgroups=2 * N_CU):
        """TFLOP/s of v_mfma_f32_32x32x16_bf16 at two wavefronts per SIMD with (fp32 FMAs, v_exp_f32 + add) per
        matrix instruction issued beside it, on random operands (what an attention pass feeds the multipliers) or on
        constant ones. (0, 0, random) is the matrix cores alone on real data: the ceiling the prefill fractions are
        also stated against."""
        t = self.torch
        outbuf = t.zeros(workgroups * 256, dtype=t.float32, device="cuda")
        st = self.C.c_void_p(t.cuda.current_stream().cuda_stream)
        flops = workgroups * 4 * iters * 32 * 32768
        out = []
        for nv, ne, rnd in mixes:
            evs = self._events(5)
            for a, b in evs:
                rc = self.lib.esp_ceiling_mfma_issue(nv, ne, rnd, workgroups, iters, self.C.c_void_p(outbuf.data_ptr()), st,
                                                     self.C.c_void_p(a.cuda_event), self.C.c_void_p(b.cuda_event))
                assert rc == 0, rc
            t.cuda.synchronize()
            ms = np.array([a.elapsed_time(b) for a, b in evs][1:])
            out.append({"valu_per_mfma": nv, "exp_per_mfma": ne, "operands": "random" if rnd else "constant",
                        "TFLOPs": round(flops / float(np.median(ms)) / 1e9, 1),
                        "ns_per_mfma_per_simd": round(float(np.median(ms)) * 1e6 / (iters * 32 * 2), 2)})
        return out


    STAGES = ("matrix instructions, operands in registers", "+ A operands read from LDS", "+ a barrier per step",
              "+ the softmax's vector work", "+ 32 KB per step staged into LDS")

    def prefill_step(self, cases=((0, 1, 1), (1, 1, 1), (2, 1, 1), (3, 1, 1), (4, 1, 1), (4, 1, 0), (1, 2, 1), (3, 2, 1), (4, 2, 1)), iters=3000):
        """TFLOP/s of the prefill kernel's step as a bare instruction stream, one ingredient more per stage, at 32
        rows per wavefront and two workgroups per compute unit (the kernels as built) or 64 rows and one, on random
        or constant operands; with the clock each launch ran at, read inside the kernel."""
        t = self.torch
        src = t.full(((4 << 20) + 65536,), 0x5b, dtype=t.uint8, device="cuda")
        st = self.C.c_void_p(t.cuda.current_stream().cuda_stream)
        out = []
        for stage, rows, rnd in cases:
            wgs = 2 * N_CU if rows == 1 else N_CU
            outbuf = t.zeros(wgs * 256, dtype=t.float32, device="cuda")
            clk = t.zeros(2 * wgs, dtype=t.int64, device="cuda")
            evs = self._events(4)
            for a, b in evs:
                rc = self.lib.esp_ceiling_prefill_step(stage, rows, rnd, wgs, iters, self.C.c_void_p(outbuf.data_ptr()), self.C.c_void_p(src.data_ptr()),
                                                       self.C.c_void_p(clk.data_ptr()), st, self.C.c_void_p(a.cuda_event), self.C.c_void_p(b.cuda_event))
                assert rc == 0, rc
            t.cuda.synchronize()
            ms = float(np.median([a.elapsed_time(b) for a, b in evs][1:]))
            ck = clk.cpu().numpy().reshape(wgs, 2).astype(np.float64)
            out.append({"stage": stage, "what": self.STAGES[stage], "rows_per_wavefront": 32 * rows, "operands": "random" if rnd else "constant",
                        "TFLOPs": round(wgs * 4 * iters * 32 * rows * 32768 / ms / 1e9, 1),
                        "clock_GHz": round(float((ck[:, 0] / (ck[:, 1] / 100e6)).mean()) / 1e9, 3)})
        return out


    SHAPES256 = ("4 wavefronts x 32 rows, one per SIMD (as built)", "8 wavefronts as 4 pairs, P through LDS",
                 "8 wavefronts x 16 rows, v_mfma_f32_16x16x32")
    LOADS256 = ("no staging loads", "64 KB per step staged behind the barrier", "one load behind each of the first 16 matrix instructions",
                "a second barrier in mid-step, each wavefront's loads beside two groups of matrix instructions of its own",
                "no staging loads, operand reads one by one behind the matrix instructions",
                "one load behind each of the first 16 matrix instructions, operand reads one by one",
                "64 KB per step staged behind the barrier, operand reads one by one")

    def prefill_step256(self, cases=((0, 0), (0, 1), (0, 2), (0, 3), (0, 4), (0, 5), (0, 6), (1, 0), (1, 1), (2, 0), (2, 1)), iters=1500):
        """The 256-dim prefill step as bare instruction streams in three shapes of the workgroup, one workgroup per
        compute unit: TFLOP/s, cycles per step (64 keys x 128 rows) and the clock, both read inside the kernel."""
        t = self.torch
        src = t.full(((8 << 20) + 65536,), 0x3c, dtype=t.uint8, device="cuda")
        st = self.C.c_void_p(t.cuda.current_stream().cuda_stream)
        out = []
        for shape, loads in cases:
            outbuf = t.zeros(N_CU * 512, dtype=t.float32, device="cuda")
            clk = t.zeros(2 * N_CU, dtype=t.int64, device="cuda")
            evs = self._events(4)
            for a, b in evs:
                rc = self.lib.esp_ceiling_prefill_step256(shape, loads, N_CU, iters, self.C.c_void_p(outbuf.data_ptr()), self.C.c_void_p(src.data_ptr()),
                                                          self.C.c_void_p(clk.data_ptr()), st, self.C.c_void_p(a.cuda_event), self.C.c_void_p(b.cuda_event))
                assert rc == 0, rc
            t.cuda.synchronize()
            ms = float(np.median([a.elapsed_time(b) for a, b in evs][1:]))
            ck = clk.cpu().numpy().reshape(N_CU, 2).astype(np.float64)
            out.append({"shape": self.SHAPES256[shape], "loads": self.LOADS256[loads],
                        "TFLOPs": round(N_CU * iters * 256 * 32768 / ms / 1e9, 1),
                        "cycles_per_step": round(float(ck[:, 0].mean()) / iters, 0),
                        "clock_GHz": round(float((ck[:, 0] / (ck[:, 1] / 100e6)).mean()) / 1e9, 3)})
        return out


def run_all(args, torch):
    """The default run: the batched paged decode as the headline (its K timed steps are the line's steps), the
    chunked causal prefill as the other half of the metric, one record per benchmark configuration (each with its
    kernel roofline, a parity spot check and a CPU baseline of its own), and the machine's measured ceilings."""
    K, W = args.steps, args.warmup
    cpu = not args.no_cpu
    # The machine's own ceilings, for orientation only (no fraction is stated against them): a plain read kernel at
    # the sizes of C2 / C5 / C4 global, and the matrix cores alone. Measured first: a GPU that has sat idle takes
    # milliseconds to leave its low-power state, more than the W warm-up steps of a 30 us pass last.
    ceil = Ceilings()
    ceilings = {"hbm_read": ceil.hbm_read(), "mfma_issue": ceil.mfma_issue()}
    w = make_workload("c2_batched_decode", args.workgroups or None, args.tables == "contiguous", args.page)
    wall, per_launch = timed_run(w, torch, K, W)
    out = headline(w, wall, per_launch, K, W)
    out["graph_replay"] = graph_replay(w, torch)
    err, n = spot_check(w)
    c2 = {"workload": w.name, "ms_per_step": out["ms_per_step"], "kernel_us_avg": out["roofline"]["kernel_us_avg"],
          "kernel_us_median": out["roofline"]["kernel_us_median"], "kernel_us_min": out["roofline"]["kernel_us_min"],
          "frac": out["roofline"]["frac"], "max_abs_err_vs_cpu": err, "rows_checked": n, "tolerance": tolerance()}
    if cpu:
        out["cpu_baseline"] = cpu_leg(w, torch)
        c2["cpu_baseline"] = out["cpu_baseline"]
    del w
    torch.cuda.empty_cache()

    # ---- the prefill half of the metric: config 3 whole (4 x (attention, merge, append)), chunk by chunk beside it
    steps_p = max(5, min(20, K // 10))
    w = make_workload("c3_chunked_prefill", args.workgroups or None, False, args.page)
    rec, pl = compact(w, torch, steps_p, 3)
    chunk = w.n_rows // pl.shape[1]
    parts = []
    for c in range(pl.shape[1]):
        pairs = chunk * c * chunk + chunk * (chunk + 1) // 2
        parts.append(part_record(f"chunk P={c * chunk}", 4 * w.HD * w.H * pairs, 1e12, MFMA_PEAK_TFLOPS, pl[:, c]))
    pre = {"metric": "prefill-attn TFLOPS", "value": rec["value"], "unit": "TFLOP/s", "ms_per_step": rec["ms_per_step"],
           "steps": steps_p, "dtype": "bf16", "config": {"workload": w.name, "rows": w.n_rows, "chunk": chunk, "H": w.H, "Hkv": w.Hkv,
                                                        "head_dim": w.HD, "page": w.bt},
           "roofline": roofline(w, pl.sum(axis=1)), "chunks": parts, "graph_replay": graph_replay(w, torch, steps=2, replays=4),
           "tolerance": tolerance()}
    if cpu:
        w.step(0)
        torch.cuda.synchronize()
        pre["cpu_baseline"] = chunked_cpu_baseline(w)
        pre["max_abs_err_vs_cpu"] = pre["cpu_baseline"]["max_abs_err_vs_gpu"]
    out["prefill"] = pre
    del w
    torch.cuda.empty_cache()

    # ---- one record per benchmark configuration
    configs = [c2]
    for name, steps in (("c1_single_decode", 50), ("c5_verify", 30), ("c4_decode_mix", 20), ("c4_prefill_mix", 5)):
        w = make_workload(name, args.workgroups or None, False, args.page)
        rec, pl = compact(w, torch, steps, 3)
        rec["graph_replay_us_per_step"] = graph_replay(w, torch, steps=4 if w.bound == "mfma" else 16, replays=4).get("us_per_step")
        if isinstance(w, LayerMix):
            hb = w.bound == "hbm"
            peak, sc = (HBM_PEAK_GBS, 1e9) if hb else (MFMA_PEAK_TFLOPS, 1e12)
            rec["layers"] = [
                part_record("sliding layer (each of 5)", w.sliding.alg_bytes if hb else w.sliding.alg_flops, sc, peak, pl[:, :5].reshape(-1)),
                part_record("global layer", w.full.alg_bytes if hb else w.full.alg_flops, sc, peak, pl[:, 5])]
            e1, n1 = spot_check(w.sliding)
            e2, n2 = spot_check(w.full)
            rec["max_abs_err_vs_cpu"], rec["rows_checked"] = max(e1, e2), n1 + n2
        else:
            rec["max_abs_err_vs_cpu"], rec["rows_checked"] = spot_check(w)
        if cpu:
            rec["cpu_baseline"] = cpu_leg(w, torch, budget_s=6.0)
        configs.append(rec)
        del w
        torch.cuda.empty_cache()
    configs.insert(2, {"workload": "c3_chunked_prefill", "ms_per_step": pre["ms_per_step"], "frac": pre["roofline"]["frac"],
                       "kernel_us_avg": pre["roofline"]["kernel_us_avg"], "kernel_us_median": pre["roofline"]["kernel_us_median"],
                       "kernel_us_min": pre["roofline"]["kernel_us_min"], "max_abs_err_vs_cpu": pre.get("max_abs_err_vs_cpu"),
                       "tolerance": pre["tolerance"], "cpu_baseline": pre.get("cpu_baseline"), "see": "prefill"})
    out["configs"] = configs
    # the decode step from the fp32 projection to O: esp_attn_prep + esp_attn_forward against esp_attn_decode_fused
    fa = argparse.Namespace(**{**vars(args), "steps": 100, "warmup": 10})
    out["decode_step"] = decode_step_fusion(fa, torch, ("c1_single_decode", "c2_batched_decode", "c4_decode_sliding"), emit=False)["configs"]
    out["prefill_step"] = prefill_step_fusion(args, torch, emit=False)
    out["ceilings"] = ceilings
    out["traffic_source"] = traffic_source()
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="all",
                    help="all (default): the batched decode as the headline, the chunked prefill, one record per benchmark "
                         "configuration and the measured ceilings; or c2_equal_<tokens> (16 equal sequences), or one of: hbm_read_ceiling, mfma_issue_ceiling, prefill_step_ceiling, prefill_step256_ceiling, decode_step_fusion, prefill_step_fusion, " + ", ".join(WORKLOADS))
    ap.add_argument("--workgroups", type=int, default=0, help="planner split target (0: ask esp_attn_plan_hint)")
    ap.add_argument("--cut-batch", action="store_true", help="experiment: let the planner cut a tile's batch keys too (esp_plan_options.cut_batch)")
    ap.add_argument("--plan-costs", default="", help="experiment: the planner's item_steps,part_steps (e.g. 3,4) instead of its own")
    ap.add_argument("--tables", default="scattered", choices=["scattered", "contiguous"],
                    help="block tables: a seeded permutation of the pool (the benchmark's definition) or address order")
    ap.add_argument("--page", type=int, default=16, help="tokens per KV block (the benchmark's definition: 16)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this path has no multi-GPU leg (run with --gpus 1)")
    if args.cut_batch:
        PLAN_TWEAK["cut_batch"] = 1
    if args.plan_costs:
        PLAN_TWEAK["item_steps"], PLAN_TWEAK["part_steps"] = (int(x) for x in args.plan_costs.split(","))

    import torch
    from espetero_amd import device
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    device.init(0)
    if args.copy_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)   # a plain copy kernel of known size: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    if args.workload == "all":
        return run_all(args, torch)
    if args.workload == "decode_step_fusion":
        return decode_step_fusion(args, torch)
    if args.workload == "prefill_step_fusion":
        return prefill_step_fusion(args, torch)
    if args.workload == "hbm_read_ceiling":
        print(json.dumps({"metric": "plain read GB/s", "unit": "GB/s", "peak": HBM_PEAK_GBS, "sizes": Ceilings().hbm_read()}), flush=True)
        return
    if args.workload == "mfma_issue_ceiling":
        print(json.dumps({"metric": "matrix cores under vector issue, TFLOP/s", "unit": "TFLOP/s", "peak": MFMA_PEAK_TFLOPS,
                          "mixes": Ceilings().mfma_issue()}), flush=True)
        return
    if args.workload == "prefill_step_ceiling":
        print(json.dumps({"metric": "the prefill kernels' step as a bare instruction stream, TFLOP/s", "unit": "TFLOP/s",
                          "peak": MFMA_PEAK_TFLOPS, "stages": Ceilings().prefill_step()}), flush=True)
        return
    if args.workload == "prefill_step256_ceiling":
        print(json.dumps({"metric": "the 256-dim prefill step as a bare instruction stream, three workgroup shapes, TFLOP/s", "unit": "TFLOP/s",
                          "peak": MFMA_PEAK_TFLOPS, "streams": Ceilings().prefill_step256()}), flush=True)
        return
    w = make_workload(args.workload, args.workgroups or None, args.tables == "contiguous", args.page)
    K, W = args.steps, args.warmup
    wall, per_launch = timed_run(w, torch, K, W)
    out = headline(w, wall, per_launch, K, W)
    if per_launch.shape[1] > 1:
        out["roofline"]["per_launch_us_median"] = [round(float(x) * 1e3, 3) for x in np.median(per_launch, axis=0)]
    out["graph_replay"] = graph_replay(w, torch)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_leg(w, torch)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
