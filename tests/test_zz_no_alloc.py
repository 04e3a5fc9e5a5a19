"""esp_attn_forward_static: the attention entry point that allocates nothing. Its partial records and
staging live in a device array the library owns; results must be those of esp_attn_forward, bit for bit,
call after call, also when a smaller pass follows a larger one in the same array."""
import numpy as np
import pytest

from espetero_amd import abi, device, host, synth

from helpers import max_abs, oracle_direct, small_case, tol_for

pytestmark = pytest.mark.gpu


def _both(case, options):
    from gpu_utils import run_case
    print(f"static vs workspace: {case.name} seqs={case.meta['seqs']} R={case.params.rows_per_tile}", flush=True)
    want = run_case(case, options)
    got = run_case(case, options, static=True)
    assert (got == want).all(), f"{case.name}: the static entry point differs from esp_attn_forward"
    err = max_abs(got, oracle_direct(case, threads=8), case.params.dtype)
    assert err <= tol_for(case.params.dtype), f"{case.name}: max abs {err}"


def test_static_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    # a split decode + verify pass (streaming kernel, merge in the kernel's tail), then a smaller one
    big = small_case(seed=71, seqs=((6000, 4), (3000, 4), (777, 4)), H=32, Hkv=4, rows_per_tile=4,
                     desc_fn=lambda M: synth.verify_desc(M, 1))
    small = small_case(seed=72, seqs=((900, 1), (40, 1)), H=32, Hkv=4, rows_per_tile=1)
    device.init(0)
    _both(big, host.options_mi355x(4, 512))
    _both(small, host.options_mi355x(1, 64))
    # prefill tiles split in two (tiled kernel: staged V and partial records in the array, merge as a dispatch), then a smaller chunk
    big = small_case(seed=73, seqs=((3000, 300),), H=10, Hkv=2, dtype=abi.ESP_BF16, rows_per_tile=128)
    small = small_case(seed=74, seqs=((100, 70),), H=10, Hkv=2, dtype=abi.ESP_BF16, rows_per_tile=128)
    _both(big, host.options_mi355x(128, 64))
    _both(small, host.options_mi355x(128, 64))


def test_static_entry_point_leaves_device_memory_as_it_found_it():
    """Free device memory as the driver reports it is the same before and after a run of static calls (every buffer
    of the passes themselves is allocated before the first reading)."""
    import torch
    from gpu_utils import dev_u16, native_pool, plan
    device.init(0)
    runs = []
    for case, wg in ((small_case(seed=76, seqs=((5000, 1), (300, 1)), H=32, Hkv=4, rows_per_tile=1), 256),
                     (small_case(seed=77, seqs=((1500, 200),), H=10, Hkv=2, dtype=abi.ESP_BF16, rows_per_tile=128), 64)):
        tiles, jobs, n_parts = plan(case, host.options_mi355x(case.params.rows_per_tile, wg))
        assert n_parts > 0
        dp = device.DevicePass(case.params, case.trees, tiles, jobs, n_parts, case.n_rows, case.blocks, case.desc, case.pos,
                               pool_blocks=case.n_blocks, static=True)
        Q = dev_u16(case.Q)
        runs.append((dp, Q, dev_u16(case.Kb), dev_u16(case.Vb), native_pool(case), torch.zeros_like(Q)))
    for dp, Q, Kb, Vb, pool, O in runs:   # first calls: whatever one-time set-up there is has happened
        dp.run(Q, Kb, Vb, pool, O)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        for dp, Q, Kb, Vb, pool, O in runs:
            dp.run(Q, Kb, Vb, pool, O)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, f"free device memory went from {free0} to {free1} over ten static calls"


def test_static_entry_point_names_its_limit():
    """A pass whose records do not fit the array is refused before anything is launched."""
    import torch
    from gpu_utils import dev_u16, native_pool, plan
    case = small_case(seed=75, seqs=((5000, 8),) * 6, H=32, Hkv=4, rows_per_tile=4)
    device.init(0)
    tiles, jobs, n_parts = plan(case, host.options_mi355x(4, 16384))
    assert device.workspace_bytes(case.params, case.n_rows, n_parts) > abi.ESP_STATIC_SCRATCH_BYTES
    dp = device.DevicePass(case.params, case.trees, tiles, jobs, n_parts, case.n_rows, case.blocks, case.desc, case.pos,
                           pool_blocks=case.n_blocks, static=True)
    Q, Kb, Vb = dev_u16(case.Q), dev_u16(case.Kb), dev_u16(case.Vb)
    O = torch.zeros_like(Q)
    with pytest.raises(abi.EspError, match="scratch"):
        dp.run(Q, Kb, Vb, native_pool(case), O)
