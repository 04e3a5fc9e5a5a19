"""The host engine's own records driving the kernels through serving histories - prefill chunks, decode
steps, forks, verify trees with hosted draft prefixes, passes that are not committed - where every pass
takes its trees / descriptors / positions / block table / copy-on-write pairs / save entries from
`KvEngine` and runs on the GPU through the C ABI, in the reference's order: block copies first
(src/model/impl/forest.h:2726-2729), attention, then the saves (forest.h:2935-2947). The CPU checker follows
in a reference-layout pool fed by the same records, and a model that knows no blocks - the list of K / V
rows every slot logically holds - is checked against both: what a tree's table exposes at attention time is
its parent's rows, and what a slot's block list reads back after the pass is the slot's rows.
Bar: attention outputs within the path's tolerance; rows and the pool bit-identical."""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, host, synth
from oracle import binding as ob

from helpers import TOL, beyond_rounding, f32, tol_for

pytestmark = pytest.mark.gpu


class Served:
    def __init__(self, H, Hkv, HD, bt, dtype, n_blocks, n_slots, seed, window=0, sliding=None):
        """sliding: (Hkv, head dim) of the sliding layer when they differ from the full layer's (Gemma 4: gemma.h:126-150)."""
        device.init(0)
        self.rng = np.random.default_rng(seed)
        self.dtype, self.n_blocks = dtype, n_blocks
        self.ap = synth.make_params(H, Hkv, HD, dtype, bt)
        self.region = n_blocks * 2 * bt * self.ap.kv_ld
        self.pool_ref = np.zeros(self.region, np.uint16)
        self.pool = torch.zeros(self.region, dtype=torch.int16, device="cuda")
        self.e = host.Engine(n_blocks, bt, n_slots)
        self.slots = [self.e.slot_alloc() for _ in range(n_slots)]
        empty = np.zeros((0, self.ap.kv_ld), np.uint16)
        self.truth = {s: (empty, empty) for s in self.slots}     # slot -> (K rows, V rows) it logically holds
        self.tol = tol_for(dtype)   # against the checker's output in the storage type
        self.max_rows = device.plan_hint3(self.ap)[2]
        # a sliding layer beside it: one ring of rb blocks per slot in a pool of its own (forest.h:2657-2700)
        self.W = window
        if window:
            self.rb = (window + bt - 1) // bt
            Hkv_s, HD_s = sliding or (Hkv, HD)
            self.ap_s = synth.make_params(H, Hkv_s, HD_s, dtype, bt, window=window, ring=self.rb)
            self.ring_region = n_slots * self.rb * 2 * bt * self.ap_s.kv_ld
            empty_s = np.zeros((0, self.ap_s.kv_ld), np.uint16)
            self.truth_s = {s: (empty_s, empty_s) for s in self.slots}   # the sliding layer has K / V rows of its own
            self.ring_ref = np.zeros(self.ring_region, np.uint16)
            self.ring = torch.zeros(self.ring_region, dtype=torch.int16, device="cuda")

    def ring_copy(self, pairs):
        pairs = np.ascontiguousarray(pairs, np.int32)
        if len(pairs):
            device.kv_copy_blocks(self.ap_s, self.ring, device.to_dev(pairs), len(pairs), 1, self.ring_region)
            ob.kv_copy_blocks(self.ap_s, self.ring_ref, pairs, 1, self.ring_region)

    def reset(self, s):
        self.e.slot_reset(s)
        self.truth[s] = (self.truth[s][0][:0], self.truth[s][1][:0])
        if self.W:
            self.truth_s[s] = (self.truth_s[s][0][:0], self.truth_s[s][1][:0])

    def fork(self, a, b):
        self.reset(b)
        self.e.slot_fork(a, b)
        self.truth[b] = self.truth[a]
        if self.W:                                                 # a fork copies the whole ring (forest.h:127-137)
            self.truth_s[b] = self.truth_s[a]
            self.ring_copy([(a * self.rb + i, b * self.rb + i) for i in range(self.rb)])

    def run(self, specs, rows_per_tile, commit=True, tag=""):
        """specs: [(parent, save, root_len, leaves, commit_chain)]. False if the engine refused the pass."""
        from gpu_utils import dev_u16, to_host_u16
        ap, e, dtype = self.ap, self.e, self.dtype
        try:
            ps = e.pass_begin([host.make_spec(parent=p, save=s, root_len=r, leaves=lv, commit_chain=cc) for p, s, r, lv, cc in specs])
        except abi.EspError as ex:
            print(f"{tag}: refused ({ex})", flush=True)
            return False
        M = ps["M"]
        print(f"{tag}: M={M} rows/tile={rows_per_tile} trees={[tuple(int(x) for x in t) for t in ps['trees']]} "
              f"cow={ps['cow'].tolist()} saves={len(ps['saves'])}", flush=True)
        bits = lambda w: ob.from_f32(self.rng.standard_normal((M, w)).astype(np.float32) * 0.5, dtype)  # noqa: E731
        Q, Kb, Vb = bits(ap.q_ld), bits(ap.kv_ld), bits(ap.kv_ld)
        blocks = ps["table"] if len(ps["table"]) else np.zeros(1, np.int32)
        if len(ps["cow"]):
            device.kv_copy_blocks(ap, self.pool, device.to_dev(np.ascontiguousarray(ps["cow"], np.int32)), len(ps["cow"]), 1, self.region)
            ob.kv_copy_blocks(ap, self.pool_ref, ps["cow"], 1, self.region)
        for t, (parent, *_) in zip(ps["trees"], specs):           # the table of every tree exposes its parent's rows
            P = int(t["P"])
            assert P == (len(self.truth[parent][0]) if parent >= 0 else 0)
            if P:
                kw, vw = ob.kv_gather(ap, self.pool_ref, blocks[int(t["table"]):], P)
                assert np.array_equal(kw, self.truth[parent][0]) and np.array_equal(vw, self.truth[parent][1]), tag
        ap.rows_per_tile = rows_per_tile
        resident, groups = device.plan_hint(ap)
        tiles, jobs, n_parts = host.plan_tiles(ps["trees"], groups, 0, None, host.options_mi355x(rows_per_tile, resident))
        dp = device.DevicePass(ap, ps["trees"], tiles, jobs, n_parts, M, blocks, ps["desc"], ps["pos"])
        Qd, Kd, Vd = dev_u16(Q), dev_u16(Kb), dev_u16(Vb)
        O = torch.zeros_like(Qd)
        dp.run(Qd, Kd, Vd, self.pool, O)
        torch.cuda.synchronize()
        want = ob.attn_direct(ap, Q, Kb, Vb, self.pool_ref, blocks, ps["desc"], ps["pos"], ps["trees"], n_threads=8)
        err = beyond_rounding(f32(to_host_u16(O).reshape(M, -1), dtype), f32(want, dtype), dtype, True)
        assert err <= self.tol, (tag, err)
        if self.W:                                                 # the same rows through the sliding layer
            rg = e.pass_rings(self.W, self.rb)
            self.ring_copy(rg["copies"])
            aps = self.ap_s
            aps.rows_per_tile = rows_per_tile
            resident, groups = device.plan_hint(aps)
            tiles, jobs, n_parts = host.plan_tiles(rg["trees"], groups, self.W, ps["pos"], host.options_mi355x(rows_per_tile, resident))
            dps = device.DevicePass(aps, rg["trees"], tiles, jobs, n_parts, M, np.zeros(1, np.int32), ps["desc"], ps["pos"])
            Qs, Kbs, Vbs = bits(aps.q_ld), bits(aps.kv_ld), bits(aps.kv_ld)
            Qsd, Ksd, Vsd = dev_u16(Qs), dev_u16(Kbs), dev_u16(Vbs)
            Os = torch.zeros_like(Qsd)
            dps.run(Qsd, Ksd, Vsd, self.ring, Os)
            torch.cuda.synchronize()
            want = ob.attn_direct(aps, Qs, Kbs, Vbs, self.ring_ref, np.zeros(1, np.int32), ps["desc"], ps["pos"], rg["trees"], n_threads=8)
            err = beyond_rounding(f32(to_host_u16(Os).reshape(M, -1), dtype), f32(want, dtype), dtype, True)
            assert err <= self.tol, (tag, "sliding", err)
            if commit and len(rg["saves"]):
                device.kv_save(aps, Ksd, Vsd, self.ring, device.to_dev(rg["saves"]), len(rg["saves"]))
                ob.kv_save(aps, Kbs, Vbs, self.ring_ref, rg["saves"])
        if not commit:
            e.pass_abort()     # the copied blocks go back to the free list; nothing a slot lists has changed
            self.check_slots(tag)
            return True
        if len(ps["saves"]):
            device.kv_save(ap, Kd, Vd, self.pool, device.to_dev(ps["saves"]), len(ps["saves"]))
            ob.kv_save(ap, Kb, Vb, self.pool_ref, ps["saves"])
        torch.cuda.synchronize()
        e.pass_commit()
        new, new_s = {}, {}
        for t, (parent, save, root_len, *_) in zip(ps["trees"], specs):
            if save >= 0:                                          # the slot takes its parent's rows and the tree's root
                pk, pv = self.truth[parent] if parent >= 0 else (Kb[:0], Vb[:0])
                b = int(t["base"])
                new[save] = (np.concatenate([pk, Kb[b:b + root_len]]), np.concatenate([pv, Vb[b:b + root_len]]))
                if self.W:
                    pk, pv = self.truth_s[parent] if parent >= 0 else (Kbs[:0], Vbs[:0])
                    new_s[save] = (np.concatenate([pk, Kbs[b:b + root_len]]), np.concatenate([pv, Vbs[b:b + root_len]]))
        self.truth.update(new)
        if self.W:
            self.truth_s.update(new_s)
        self.last = (ps, specs, Kb, Vb)
        self.check_slots(tag)
        return True

    def accept(self, slot, n):
        """Verify-commit: the first n chain rows the last pass kept for `slot` join it (forest.h:4846-4861)."""
        ps, specs, Kb, Vb = self.last
        (t, spec), = [(t, sp) for t, sp in zip(ps["trees"], specs) if sp[1] == slot]
        assert self.e.slot_chain(slot) == spec[4] and n <= spec[4]
        self.e.chain_commit(slot, n)
        print(f"accept {n} of {spec[4]} chain rows of slot {slot}", flush=True)
        b = int(t["base"]) + spec[2]                               # the chain's rows follow the root's
        self.truth[slot] = (np.concatenate([self.truth[slot][0], Kb[b:b + n]]), np.concatenate([self.truth[slot][1], Vb[b:b + n]]))
        self.check_slots(f"accept {n} of slot {slot}")

    def check_slots(self, tag):
        for s in self.slots:
            n = len(self.truth[s][0])
            assert self.e.slot_len(s) == n, (tag, s)
            if n:
                kw, vw = ob.kv_gather(self.ap, self.pool_ref, self.e.slot_blocks(s), n)
                assert np.array_equal(kw, self.truth[s][0]) and np.array_equal(vw, self.truth[s][1]), (tag, s)
            if n and self.W:                                       # the ring reads back what the slot's next row can see
                lo = max(0, n - self.W + 1)
                order = [s * self.rb + i % self.rb for i in range((n + self.ap.bt - 1) // self.ap.bt)]
                kw, vw = ob.kv_gather(self.ap_s, self.ring_ref, np.array(order, np.int32), n)
                assert np.array_equal(kw[lo:], self.truth_s[s][0][lo:]) and np.array_equal(vw[lo:], self.truth_s[s][1][lo:]), (tag, s, "ring")

    def finish(self):
        """The device pool holds what the reference-layout pool holds, block for block, and every slot reads back
        through the device's gather as its rows."""
        from gpu_utils import to_host_u16
        back = torch.zeros_like(self.pool)
        device.kv_relayout(self.ap, self.pool, abi.ESP_LAYOUT_NATIVE, back, abi.ESP_LAYOUT_REFERENCE, self.n_blocks)
        torch.cuda.synchronize()
        assert np.array_equal(to_host_u16(back), self.pool_ref)
        if self.W:
            back = torch.zeros_like(self.ring)
            device.kv_relayout(self.ap_s, self.ring, abi.ESP_LAYOUT_NATIVE, back, abi.ESP_LAYOUT_REFERENCE, len(self.slots) * self.rb)
            torch.cuda.synchronize()
            assert np.array_equal(to_host_u16(back), self.ring_ref)
        for s in self.slots:
            n = len(self.truth[s][0])
            if not n:
                continue
            Kg = torch.zeros(n * self.ap.kv_ld, dtype=torch.int16, device="cuda")
            Vg = torch.zeros_like(Kg)
            device.kv_gather(self.ap, self.pool, device.to_dev(np.ascontiguousarray(self.e.slot_blocks(s), np.int32)), n, Kg, Vg)
            torch.cuda.synchronize()
            assert np.array_equal(to_host_u16(Kg).reshape(n, -1), self.truth[s][0])
            assert np.array_equal(to_host_u16(Vg).reshape(n, -1), self.truth[s][1])


# the last: Gemma 4's two layer kinds off the same records - full layers of 512-dim heads on few KV heads, sliding layers
# of 256-dim heads on more (gemma.h:126-150)
@pytest.mark.parametrize("H,Hkv,HD,bt,dtype,window,sliding", [(8, 2, 128, 16, abi.ESP_F16, 0, None), (8, 1, 512, 32, abi.ESP_F16, 0, None),
                                                              (6, 3, 256, 64, abi.ESP_BF16, 100, None),
                                                              (16, 2, 512, 16, abi.ESP_F16, 72, (8, 256))])
def test_engine_records_drive_the_kernels_through_a_serving_history(H, Hkv, HD, bt, dtype, window, sliding):
    sv = Served(H, Hkv, HD, bt, dtype, 96, 4, H + HD, window=window, sliding=sliding)
    A, B, Cc, D = sv.slots
    e = sv.e
    G = H // Hkv
    sv.run([(-1, A, 100, (), 0), (-1, B, 57, (), 0)], sv.max_rows, tag="prefill A, B")
    for s in range(3):
        sv.run([(A, A, 1, (), 0), (B, B, 1, (), 0)], 1, tag=f"decode {s}")
    sv.fork(A, Cc)
    drafts = [5, 6, 7]
    leaves = [drafts[:i + 1] for i in range(3)]
    rows_verify = 4 if HD < 512 else max(1, 16 // G)       # what the streaming kernel packs at this head dim
    chain = 0 if sv.W else 3                                # the reference keeps no chain on models with sliding layers (forest.h:2237)
    sv.run([(Cc, Cc, 1, leaves, chain), (A, A, 1, (), 0)], rows_verify, tag="verify C (fork of A: copy on write) + decode A")
    if chain:
        sv.accept(Cc, 2)                                    # two of the three drafts accepted
    sv.run([(B, -1, 2, [[1, 2], [1, 3, 4], [9]], 0)], 8 if HD < 512 else max(1, 16 // G), commit=False,
           tag="wide verify tree on B, not committed")
    sv.run([(B, B, 45, (), 0), (A, D, 20, (), 0)], sv.max_rows, tag="chunk on B + A continued into D")
    sv.run([(s_, s_, 1, (), 0) for s_ in (A, B, Cc, D)], 1, tag="decode all four")
    # the verify pass commits its root token; the accepted drafts come on top
    assert (e.slot_len(A), e.slot_len(B), e.slot_len(Cc), e.slot_len(D)) == (105, 106, 105 + (2 if chain else 0), 125)
    sv.finish()


def _random_leaves(rng):
    """A few draft token lists over a small alphabet, so that prefixes are shared and hosted once."""
    return [[int(x) for x in rng.integers(1, 4, int(rng.integers(1, 5)))] for _ in range(int(rng.integers(1, 5)))]


@pytest.mark.parametrize("seed", range(6))
def test_random_serving_histories(seed):
    """Random passes of up to three trees (chunks, decode rows, verify trees; in place, into another slot, from
    nothing), forks and resets in between, one pass in four not committed, a pool small enough that some
    passes are refused; geometry, block size, tile height and the sliding layer's window drawn per history."""
    rng = np.random.default_rng(4000 + seed)
    H, Hkv, HD = [(8, 2, 128), (4, 4, 128), (16, 2, 256), (6, 3, 256), (8, 1, 512), (4, 2, 512)][seed % 6]
    bt = int(rng.choice([16, 32, 64]))
    dtype = abi.ESP_F16 if seed % 2 == 0 else abi.ESP_BF16
    n_slots = 4
    window = 0 if HD == 512 or seed == 0 else int(rng.integers(20, 200))   # 512-dim heads are the layers without a window
    sv = Served(H, Hkv, HD, bt, dtype, int(rng.integers(24, 64)) * 64 // bt, n_slots, 5000 + seed, window)
    heights = [r for r in (1, 2, 4, 8, 16, sv.max_rows) if r <= sv.max_rows]
    n_passes = 0
    for step in range(30):
        op = rng.choice(["pass", "fork", "reset"], p=[0.8, 0.15, 0.05])
        if op == "fork":
            a, b = (int(x) for x in rng.choice(sv.slots, 2, replace=False))
            sv.fork(a, b)
            continue
        if op == "reset":
            sv.reset(int(rng.choice(sv.slots)))
            continue
        dsts = [int(x) for x in rng.choice(sv.slots, int(rng.integers(1, 4)), replace=False)]
        specs = []
        for d in dsts:
            kind = rng.choice(["inplace", "from", "fresh"], p=[0.75, 0.2, 0.05])
            parent = d if len(sv.truth[d][0]) and kind != "fresh" else -1
            if kind == "from":
                other = int(rng.choice(sv.slots))
                if len(sv.truth[other][0]) and other != d and other not in dsts:   # a parent that another tree rewrites is left out
                    parent = other
            if parent != d:
                sv.reset(d)
            shape = rng.choice(["chunk", "decode", "verify"]) if parent >= 0 else "chunk"
            if shape == "chunk":
                specs.append((parent, d, int(rng.integers(2, 90)), (), 0))
            elif shape == "decode":
                specs.append((parent, d, 1, (), 0))
            else:
                leaves = _random_leaves(rng)
                chain = int(rng.integers(0, 2)) if parent == d and not sv.W else 0   # kept chains: in place, no sliding layers
                if chain:                                          # leaves [0, k) one chain: prefixes of one draft
                    draft = [int(x) for x in rng.integers(1, 4, int(rng.integers(1, 4)))]
                    leaves = [draft[:i + 1] for i in range(len(draft))] + [l for l in leaves if l[0] != draft[0]]
                    chain = len(draft)
                specs.append((parent, d, int(rng.integers(1, 3)), leaves, chain))
        rows = 1 if all(s[2] == 1 and not s[3] for s in specs) else int(rng.choice(heights))
        commit = rng.integers(0, 4) != 0
        ran = sv.run(specs, rows, commit=commit, tag=f"seed {seed} step {step}")
        n_passes += ran
        if ran and commit:
            for sp in specs:
                if sp[4] and rng.integers(0, 3):
                    sv.accept(sp[1], int(rng.integers(0, sp[4] + 1)))
    assert n_passes >= 10
    sv.finish()


@pytest.mark.parametrize("H,Hkv,HD,M,rows_per_tile,dtype", [
    (4, 2, 128, 4, 4, abi.ESP_F16),      # streaming kernel: the root's rows packed into one column tile
    (8, 1, 128, 3, 4, abi.ESP_BF16),     # 24 packed rows: two column tiles
    (4, 2, 128, 150, 128, abi.ESP_BF16),  # tiled kernel, two row tiles
    (4, 2, 256, 70, 128, abi.ESP_F16),
    (2, 1, 512, 40, 64, abi.ESP_F16),
])
def test_noncausal_root_through_the_engine(H, Hkv, HD, M, rows_per_tile, dtype):
    """A noncausal root (src/model/impl/forest.h:2402-2403; mask rule kernels/40_attention.metal:104-113, :220): the
    engine describes every row as seeing the whole root, and both kernel families then give dense bidirectional
    attention - held against the checker and against a float64 softmax that knows no mask."""
    from gpu_utils import dev_u16, to_host_u16
    device.init(0)
    rng = np.random.default_rng(5)
    e = host.Engine(8, 16, 2)
    ps = e.pass_begin([host.make_spec(root_len=M, noncausal=1)])
    assert ps["M"] == M and (ps["desc"][:, 2] == M).all()
    ap = synth.make_params(H, Hkv, HD, dtype, 16, rows_per_tile=rows_per_tile)
    bits = lambda w: ob.from_f32(rng.standard_normal((M, w)).astype(np.float32) * 0.5, dtype)  # noqa: E731
    Q, Kb, Vb = bits(ap.q_ld), bits(ap.kv_ld), bits(ap.kv_ld)
    resident, groups = device.plan_hint(ap)
    tiles, jobs, n_parts = host.plan_tiles(ps["trees"], groups, 0, None, host.options_mi355x(rows_per_tile, resident))
    blocks = np.zeros(1, np.int32)
    pool = torch.zeros(8 * 2 * 16 * ap.kv_ld, dtype=torch.int16, device="cuda")
    dp = device.DevicePass(ap, ps["trees"], tiles, jobs, n_parts, M, blocks, ps["desc"], ps["pos"], pool_blocks=8)
    Qd = dev_u16(Q)
    O = torch.zeros_like(Qd)
    print(f"noncausal root: H={H} Hkv={Hkv} HD={HD} M={M} rows/tile={rows_per_tile} tiles={len(tiles)}", flush=True)
    dp.run(Qd, dev_u16(Kb), dev_u16(Vb), pool, O)
    torch.cuda.synchronize()
    e.pass_abort()
    got = f32(to_host_u16(O).reshape(M, -1), dtype).astype(np.float64)
    want = ob.attn_direct(ap, Q, Kb, Vb, np.zeros(8 * 2 * 16 * ap.kv_ld, np.uint16), blocks, ps["desc"], ps["pos"], ps["trees"], n_threads=4)
    assert beyond_rounding(got, f32(want, dtype), dtype, True) <= tol_for(dtype)
    q = f32(Q, dtype).astype(np.float64).reshape(M, H, HD)
    k = f32(Kb, dtype).astype(np.float64).reshape(M, Hkv, HD)
    v = f32(Vb, dtype).astype(np.float64).reshape(M, Hkv, HD)
    dense = np.zeros((M, H, HD))
    for h in range(H):
        s = q[:, h] @ k[:, h // (H // Hkv)].T * ap.scale
        w = np.exp(s - s.max(axis=1, keepdims=True))
        dense[:, h] = (w / w.sum(axis=1, keepdims=True)) @ v[:, h // (H // Hkv)]
    assert beyond_rounding(got, dense.reshape(M, -1), dtype, False) <= TOL


def test_checkpoint_file_reloaded_through_slot_adopt_decodes_identically(tmp_path):
    """save -> load -> decode through the engine (src/model/model.mm:629-752): a slot filled by a prefill pass is
    exported to a checkpoint file, the file is loaded into a slot the engine adopts (fresh blocks, same length and
    next position), and a decode step on the adopted slot gives the bits of the same step on the original."""
    from gpu_utils import dev_u16, to_host_u16
    sv = Served(8, 2, 128, 16, abi.ESP_F16, 64, 3, seed=17)
    a, b, c = sv.slots
    sv.e.slot_free(c)                                              # slot_adopt takes a free slot
    sv.slots = [a, b]
    assert sv.run([(-1, a, 77, [], 0)], 128, tag="prefill 77 rows into a")
    ap, e = sv.ap, sv.e
    blocks = e.slot_blocks(a)
    nb, blk = len(blocks), 2 * ap.bt * ap.kv_ld
    out = torch.zeros(1, nb, blk, dtype=torch.int16, device="cuda")
    device.kv_export_blocks(ap, sv.pool, device.to_dev(blocks), nb, out[0])
    torch.cuda.synchronize()
    path = tmp_path / "a.ckpt"
    host.slot_file_save(path, e.slot_len(a), e.slot_next_pos(a), 1, to_host_u16(out))
    got = host.slot_file_load(path, ap.bt)
    assert got is not None and got["len"] == 77
    s = e.slot_adopt(got["len"], got["next_pos"], got["n_blocks"])
    assert s == c and e.slot_len(s) == 77 and e.slot_next_pos(s) == e.slot_next_pos(a)
    nblocks = e.slot_blocks(s)
    assert not set(nblocks.tolist()) & set(blocks.tolist())
    device.kv_import_blocks(ap, dev_u16(got["kv"].view(np.uint16).reshape(nb, blk)), device.to_dev(nblocks), nb, sv.pool)
    torch.cuda.synchronize()
    rng = np.random.default_rng(3)
    bits = lambda w: ob.from_f32(rng.standard_normal((1, w)).astype(np.float32) * 0.5, ap.dtype)  # noqa: E731
    Q, Kb, Vb = dev_u16(bits(ap.q_ld)), dev_u16(bits(ap.kv_ld)), dev_u16(bits(ap.kv_ld))
    ap.rows_per_tile = 1
    resident, groups = device.plan_hint(ap)
    outs = []
    for slot in (a, s):
        ps = e.pass_begin([host.make_spec(parent=slot, save=slot, root_len=1)])
        tiles, jobs, n_parts = host.plan_tiles(ps["trees"], groups, 0, None, host.options_mi355x(1, resident))
        dp = device.DevicePass(ap, ps["trees"], tiles, jobs, n_parts, 1, ps["table"], ps["desc"], ps["pos"], pool_blocks=64)
        O = torch.zeros_like(Q)
        dp.run(Q, Kb, Vb, sv.pool, O)
        device.kv_save(ap, Kb, Vb, sv.pool, device.to_dev(ps["saves"]), len(ps["saves"]))
        torch.cuda.synchronize()
        e.pass_commit()
        outs.append(O)
    assert torch.equal(outs[0], outs[1]) and bool(outs[0].any())
    assert e.slot_len(a) == e.slot_len(s) == 78
