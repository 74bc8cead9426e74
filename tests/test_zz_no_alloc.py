"""mi355_sage_sdpa_bf16_static: the entry point that allocates nothing (its intermediates live in
a buffer that is part of the loaded library).  Same bits as mi355_sage_sdpa_bf16 on two calls in a
row, the second with a smaller input; the device's free memory does not move across a call; the
call can be recorded into a HIP graph (an allocation would end the capture with an error);
problems beyond the buffer are refused."""
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

    def call():
        rc = L.mi355_sage_sdpa_bf16_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(), w.B, w.H, w.S, w.S,
                                           w.D, w.scale, st, st, st, st, 0, 0, 0, 0, 0, H.stream(), variant)
        assert rc == 0, rc
        torch.cuda.synchronize()

    call()              # (the first call on a device looks the buffer's address up)
    # free memory of the DEVICE, as the driver reports it: an allocation by the library itself
    # would show here, where torch's own counters only see torch's allocator
    free_before = torch.cuda.mem_get_info()[0]
    got.zero_()
    call()
    assert torch.cuda.mem_get_info()[0] >= free_before
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


@pytest.mark.parametrize("variant", [0, 1])
def test_static_scratch_entry_point_inside_a_graph_capture(variant):
    """While a stream is being captured every allocating call fails and invalidates the capture;
    this entry point is recorded without one, and the replays reproduce the eager result."""
    import torch
    import gpu_harness as H
    L = _lib.lib()
    w = WORKLOADS[2].scaled(B=1, H=2, S=700)
    q0, k0, v0 = (H.dev_bf16(x) for x in make_inputs(w))
    q, k, v = q0.clone(), k0.clone(), v0.clone()
    o = torch.empty_like(q)
    st = _lib.strides_bhnd(w.S, w.H, w.D)

    def call(out):
        rc = L.mi355_sage_sdpa_bf16_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), w.B, w.H, w.S, w.S,
                                           w.D, w.scale, st, st, st, st, 0, 0, 0, 0, 0,
                                           torch.cuda.current_stream().cuda_stream, variant)
        assert rc == 0, rc

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        call(o)                                              # the address look-up happens outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        call(o)
    for rep in range(3):
        q.copy_(torch.roll(q0, rep, dims=1))
        k.copy_(k0 * (1.0 + 0.5 * rep))
        junk = (v.float() * 2.0).sum()
        torch.cuda.synchronize()
        o.zero_()
        g.replay()
        torch.cuda.synchronize()
        eager = torch.empty_like(o)
        call(eager)
        torch.cuda.synchronize()
        assert torch.isfinite(junk)
        np.testing.assert_array_equal(H.to_bits(o), H.to_bits(eager))


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
