"""The host engine's own records driving the kernels: a small serving history (prefill of two sequences,
decode steps, a fork, a verify tree with hosted draft prefixes beside a decode, a further chunk) where every
pass takes its trees / descriptors / positions / block table / copy-on-write pairs / save entries from
`KvEngine` and runs on the GPU through the C ABI. The CPU checker follows in a reference-layout pool fed by
the same records. Bar: attention outputs within the path's tolerance; the pool bit-identical at the end."""
import numpy as np
import pytest
import torch

from espetero_amd import abi, device, host, synth
from oracle import binding as ob

from helpers import f32

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("H,Hkv,HD,bt,dtype", [(8, 2, 128, 16, abi.ESP_F16), (8, 1, 512, 32, abi.ESP_F16), (6, 3, 256, 64, abi.ESP_BF16)])
def test_engine_records_drive_the_kernels_through_a_serving_history(H, Hkv, HD, bt, dtype):
    from gpu_utils import dev_u16, to_host_u16
    device.init(0)
    rng = np.random.default_rng(H + HD)
    n_blocks = 96
    ap = synth.make_params(H, Hkv, HD, dtype, bt)
    region = n_blocks * 2 * bt * ap.kv_ld
    pool_ref = np.zeros(region, np.uint16)
    pool = torch.zeros(region, dtype=torch.int16, device="cuda")
    e = host.Engine(n_blocks, bt, 4)
    A, B, Cc, D = (e.slot_alloc() for _ in range(4))
    tol = 2e-3 if dtype == abi.ESP_F16 else 4e-3
    tiled_rows = device.plan_hint3(ap)[2]

    def run(specs, rows_per_tile, commit=True, tag=""):
        ps = e.pass_begin(specs)
        M = ps["M"]
        print(f"{tag}: M={M} trees={[tuple(int(x) for x in t) for t in ps['trees']]} cow={ps['cow'].tolist()} saves={len(ps['saves'])}", flush=True)
        bits = lambda w: ob.from_f32(rng.standard_normal((M, w)).astype(np.float32) * 0.5, dtype)  # noqa: E731
        Q, Kb, Vb = bits(ap.q_ld), bits(ap.kv_ld), bits(ap.kv_ld)
        blocks = ps["table"] if len(ps["table"]) else np.zeros(1, np.int32)
        ap.rows_per_tile = rows_per_tile
        resident, groups = device.plan_hint(ap)
        tiles, jobs, n_parts = host.plan_tiles(ps["trees"], groups, 0, None, host.options_mi355x(rows_per_tile, resident))
        dp = device.DevicePass(ap, ps["trees"], tiles, jobs, n_parts, M, blocks, ps["desc"], ps["pos"])
        Qd, Kd, Vd = dev_u16(Q), dev_u16(Kb), dev_u16(Vb)
        O = torch.zeros_like(Qd)
        dp.run(Qd, Kd, Vd, pool, O)
        torch.cuda.synchronize()
        want = ob.attn_direct(ap, Q, Kb, Vb, pool_ref, blocks, ps["desc"], ps["pos"], ps["trees"], n_threads=8)
        err = float(np.abs(f32(to_host_u16(O).reshape(M, -1), dtype) - f32(want, dtype)).max())
        assert err <= tol, (tag, err)
        if not commit:
            e.pass_abort()
            return
        if len(ps["cow"]):
            device.kv_copy_blocks(ap, pool, device.to_dev(np.ascontiguousarray(ps["cow"], np.int32)), len(ps["cow"]), 1, region)
            ob.kv_copy_blocks(ap, pool_ref, ps["cow"], 1, region)
        if len(ps["saves"]):
            device.kv_save(ap, Kd, Vd, pool, device.to_dev(ps["saves"]), len(ps["saves"]))
            ob.kv_save(ap, Kb, Vb, pool_ref, ps["saves"])
        torch.cuda.synchronize()
        e.pass_commit()

    run([host.make_spec(save=A, root_len=100), host.make_spec(save=B, root_len=57)], tiled_rows, tag="prefill A, B")
    for s in range(3):
        run([host.make_spec(parent=A, save=A, root_len=1), host.make_spec(parent=B, save=B, root_len=1)], 1, tag=f"decode {s}")
    e.slot_fork(A, Cc)
    drafts = [5, 6, 7]
    leaves = [drafts[:i + 1] for i in range(3)]
    G = H // Hkv
    rows_verify = 4 if HD < 512 else max(1, 16 // G)       # what the streaming kernel packs at this head dim
    run([host.make_spec(parent=Cc, save=Cc, root_len=1, leaves=leaves, commit_chain=3), host.make_spec(parent=A, save=A, root_len=1)],
        rows_verify, tag="verify C (fork of A: copy on write) + decode A")
    run([host.make_spec(parent=B, root_len=2, leaves=[[1, 2], [1, 3, 4], [9]])], 8 if HD < 512 else max(1, 16 // G), commit=False,
        tag="wide verify tree on B, not committed")
    run([host.make_spec(parent=B, save=B, root_len=45), host.make_spec(parent=A, save=D, root_len=20)], tiled_rows,
        tag="chunk on B + A continued into D")
    run([host.make_spec(parent=s_, save=s_, root_len=1) for s_ in (A, B, Cc, D)], 1, tag="decode all four")
    assert (e.slot_len(A), e.slot_len(B), e.slot_len(Cc), e.slot_len(D)) == (105, 106, 105, 125)   # the verify pass commits its root token only
    # the device pool holds what the reference-layout pool holds, block for block
    back = torch.zeros_like(pool)
    device.kv_relayout(ap, pool, abi.ESP_LAYOUT_NATIVE, back, abi.ESP_LAYOUT_REFERENCE, n_blocks)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_u16(back), pool_ref)
