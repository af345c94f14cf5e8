"""`dew_moe_permute_static`, the entry point that allocates nothing, against `dew_moe_permute` on the same inputs:
integer outputs, so every value must be equal. Two calls in a row share the library's scratch array, the second on a
smaller input; then one that fits a single block (no scratch) and one the array cannot hold (refused by name)."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def plan_like(ops, slots, experts):
    device = torch.device("cuda:0")
    fill = lambda n: torch.full((n,), -7, dtype=torch.int32, device=device)
    return ops.Plan(order=fill(slots), rows=fill(slots), sizes=fill(experts), offsets=fill(experts + 1))


def test_the_no_allocation_sort_equals_the_workspace_sort_on_two_calls_in_a_row():
    from dew_amd import _lib, ops

    ops.device_check()
    rng = np.random.default_rng(5)
    first = True
    for tokens, k, experts in [(8192, 8, 256), (3000, 6, 200), (1500, 4, 64), (200, 2, 8)]:   # 32, 9, 3 blocks; then one block
        ids = rng.integers(0, experts, size=(tokens, k)).astype(np.int32)
        ids[ids == 1] = 2                                  # an empty expert
        ids[rng.random(ids.shape) < 0.01] = experts        # a few dropped slots: they sort last
        indices = torch.from_numpy(ids).cuda()
        want = ops.sort_by_expert(indices, experts)
        held = plan_like(ops, tokens * k, experts)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        got = ops.sort_by_expert_into(indices, experts, held)
        torch.cuda.synchronize()
        if not first:   # (the first launch of a kernel may load its code object; after it the device's free memory stays)
            assert torch.cuda.mem_get_info()[0] >= free_before
        first = False
        for field in ("sizes", "offsets", "order", "rows"):
            assert torch.equal(getattr(got, field), getattr(want, field)), (tokens, k, experts, field)
    # beyond the array: 2^21 slots over 1024 experts need 8 MiB of counts
    lib = _lib.library()
    assert lib.dew_moe_permute_workspace_bytes(1 << 21, 1024) > (1 << 20)
    dummy = torch.zeros(16, dtype=torch.int32, device="cuda:0")
    code = lib.dew_moe_permute_static(dummy.data_ptr(), 1 << 20, 2, 1024, dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(),
                                      dummy.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert code == 1 and b"use dew_moe_permute with a workspace" in lib.dew_moe_last_error()
