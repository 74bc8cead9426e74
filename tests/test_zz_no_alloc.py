"""mi355_sage_sdpa_bf16_static: the entry point that allocates nothing (its intermediates live in
a buffer that is part of the loaded library).  Same bits as mi355_sage_sdpa_bf16 on two calls in a
row, the second with a smaller input; problems beyond the buffer are refused."""
import numpy as np
import pytest

from mojodiffusion_amd import _lib
from mojodiffusion_amd.workloads import WORKLOADS, make_inputs

pytestmark = pytest.mark.gpu


def _both(w, variant):
    import torch
    import gpu_harness as H
    L = _lib.lib()
    q, k, v = (H.dev_bf16(x) for x in make_inputs(w))
    st = _lib.strides_bhnd(w.S, w.H, w.D)
    want, got = torch.zeros_like(q), torch.zeros_like(q)
    rc = L.mi355_sage_sdpa_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), want.data_ptr(), w.B, w.H, w.S, w.S, w.D,
                                w.scale, st, st, st, st, 0, 0, 0, 0, 0, H.stream(), variant, None, 0)
    assert rc == 0, rc
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = L.mi355_sage_sdpa_bf16_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(), w.B, w.H, w.S, w.S, w.D,
                                       w.scale, st, st, st, st, 0, 0, 0, 0, 0, H.stream(), variant)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return H.to_bits(got), H.to_bits(want)


@pytest.mark.parametrize("variant", [0, 1])
def test_static_scratch_entry_point_matches_the_workspace_one(variant):
    L = _lib.lib()
    assert L.mi355_sage_static_scratch_bytes() == 16 << 20
    big = WORKLOADS[2].scaled(B=1, H=4, S=1500)
    small = WORKLOADS[2].scaled(B=2, H=2, S=333)
    assert L.mi355_sage_workspace_bytes(big.B, big.H, big.S, big.S, big.D, variant) <= 16 << 20
    for w in (big, small, big):                        # the buffer keeps the previous call's contents
        got, want = _both(w, variant)
        np.testing.assert_array_equal(got, want)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    import torch
    import gpu_harness as H
    L = _lib.lib()
    w = WORKLOADS[2]                                    # 55 MiB of intermediates
    assert L.mi355_sage_workspace_bytes(w.B, w.H, w.S, w.S, w.D, 0) > 16 << 20
    x = torch.zeros((1, w.S, w.H, w.D), dtype=torch.bfloat16, device="cuda")
    st = _lib.strides_bhnd(w.S, w.H, w.D)
    rc = L.mi355_sage_sdpa_bf16_static(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), w.B, w.H, w.S, w.S, w.D,
                                       w.scale, st, st, st, st, 0, 0, 0, 0, 0, H.stream(), 0)
    assert rc == -3, rc
