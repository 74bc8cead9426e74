"""GPU tests of the attention kernel's split scheduling: the (row tile, key tile) steps of a launch
cut into equal spans for a fixed number of workgroups that hand partial results (unnormalised
accumulators, reference maxima, row sums) to each other.  Forced on small shapes, where the CPU
checker is fast, over span lengths that give whole tiles, tiles in two and in many pieces and
empty spans; and on a shape that turns it on by itself.  Bars as for the plain schedule: max-abs
<= 2e-2 against the CPU checker, cosine >= 0.999 against the fp32 referee; against the plain
schedule the outputs may differ by the rounding of the probabilities only."""
import numpy as np
import pytest

from mojodiffusion_amd import _lib
from mojodiffusion_amd.workloads import WORKLOADS, make_inputs, bf16_bits_to_f32

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
COS = 0.999


@pytest.fixture
def split():
    L = _lib.lib()

    def set_mode(mode):
        assert L.mi355_sage_set_attn_split(mode) == 0
    yield set_mode
    L.mi355_sage_set_attn_split(0)


def _close_to_plain(got_bits, plain_bits):
    """Same quantized operands, same products; only the reference maximum a probability was
    rounded against differs between the schedules."""
    a, b = bf16_bits_to_f32(got_bits), bf16_bits_to_f32(plain_bits)
    assert np.isfinite(a).all()
    np.testing.assert_allclose(a, b, atol=6e-3, rtol=1.6e-2)
    assert (got_bits == plain_bits).mean() > 0.5          # most values round to the same bf16 anyway


@pytest.mark.parametrize("wid,variant,S,groups", [(2, 0, 1100, 24), (2, 0, 1100, 64), (2, 0, 1100, 8), (2, 0, 700, 64),
                                                  (3, 0, 333, 1024), (1, 0, 1024, 40), (1, 0, 520, 16),
                                                  (2, 0, 50, 16), (1, 0, 64, 24), (2, 0, 2000, 8), (1, 0, 2000, 200)])
def test_forced_split_against_checker_and_plain_schedule(oracle, split, wid, variant, S, groups):
    import gpu_harness as H
    from test_gpu_attn import _one_shot
    w = WORKLOADS[wid].scaled(B=2, H=3, S=S)
    q, k, v = make_inputs(w)
    blkq = 128 if variant == 0 else 32
    split(-1)
    plain = _one_shot(q, k, v, w.scale, variant)
    split(groups)
    got = _one_shot(q, k, v, w.scale, variant)
    _close_to_plain(got, plain)
    _, want32 = oracle.sdpa_bf16(q, k, v, w.scale, variant=variant, blkq=blkq, blkk=64)
    cos, mx = H.cos_maxabs(bf16_bits_to_f32(got), want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k), bf16_bits_to_f32(v), w.scale)
    cos_ref, _ = H.cos_maxabs(bf16_bits_to_f32(got), ref)
    assert cos_ref >= COS, cos_ref
    # the schedule, not the moment, decides the bits: a second call repeats them
    np.testing.assert_array_equal(_one_shot(q, k, v, w.scale, variant), got)


@pytest.mark.parametrize("variant", [0, 1])
def test_forced_split_stats_masks_and_rectangular(oracle, split, variant):
    """Stats, a masked key range, trailing padding keys, an additive mask and N_q != N_kv through
    the split schedule: each against the plain schedule, Stats also against the CPU checker."""
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    w = WORKLOADS[2].scaled(B=2, H=2, S=896)
    q, k, v = make_inputs(w)
    q = np.ascontiguousarray(q[:, :700])                               # N_q = 700, N_kv = 896
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    rng = np.random.default_rng(5)
    bias = torch.from_numpy(rng.standard_normal((w.B, w.H, 700, 896)).astype(np.float32)).cuda().to(torch.bfloat16)

    def run():
        fwd = A.sdpa_flash_train_fwd_rect(qd, kd, vd, w.scale, variant)
        km = A.sdpa_qwen_keymask(kd, kd, vd, 300, 120, w.scale, variant)            # keys [120, 300) masked
        pad = A.sdpa_flash_fwd_padmask(kd, kd, vd, 777, w.scale, variant)
        add = A.sdpa_cross_masked(qd, kd, vd, bias, w.scale, variant)
        torch.cuda.synchronize()
        return [H.to_bits(fwd.o), fwd.stats.cpu().numpy(), H.to_bits(km), H.to_bits(pad.o[:, :777]), H.to_bits(add)]

    split(-1)
    plain = run()
    for groups in (24, 56):
        split(groups)
        got = run()
        for i in (0, 2, 3, 4):
            _close_to_plain(got[i], plain[i])
        np.testing.assert_allclose(got[1], plain[1], atol=1e-3)
    blkq = 128 if variant == 0 else 32
    _, want32, want_stats = oracle.sdpa_bf16(q, k, v, w.scale, variant=variant, blkq=blkq, blkk=64, want_stats=True)
    cos, mx = H.cos_maxabs(bf16_bits_to_f32(got[0]), want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)
    np.testing.assert_allclose(got[1][..., 0], want_stats, atol=2e-3 if variant == 0 else 1e-2)


def test_shape_that_splits_by_itself(split):
    """264 row tiles on 256 compute units would run in two rounds, the second almost empty: the
    library splits such a shape without being told.  The one-shot call and the stage pipeline take
    the same decision (same bits); the result agrees with the plain schedule and the fp32 referee."""
    import torch
    import gpu_harness as H
    from test_gpu_attn import _one_shot
    L = _lib.lib()
    w = WORKLOADS[1].scaled(B=1, H=33, S=2048)
    assert L.mi355_sage_workspace_bytes(w.B, w.H, w.S, w.S, w.D, 0) > \
        L.mi355_sage_workspace_bytes(w.B, 32, w.S, w.S, w.D, 0) * 33 // 32 + (1 << 20)   # hand-over slots included
    q, k, v = make_inputs(w)
    got = _one_shot(q, k, v, w.scale, 0)
    g = H.quant_qk(q, k, w.scale, 128, 64, True)["dev"]
    gv = H.quant_v(v, 0)["dev"]
    staged, _ = H.attn_fwd(g["q8"], g["qscale"], 128, g["k8"], g["kscale"], 64, gv["vq"], None, 0, w.S, w.S)
    np.testing.assert_array_equal(got, staged)
    split(-1)
    plain = _one_shot(q, k, v, w.scale, 0)
    assert not np.array_equal(got, plain)                  # it really was another schedule
    _close_to_plain(got, plain)
    qd, kd, vd = (H.dev_bf16(x).float().permute(0, 2, 1, 3) for x in (q, k, v))
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, scale=w.scale).permute(0, 2, 1, 3)
    cos, mx = H.cos_maxabs(bf16_bits_to_f32(got), ref.cpu().numpy())
    assert cos >= COS, (cos, mx)


def test_split_call_in_a_hip_graph(split):
    """The hand-over flags are cleared by a kernel of the same call, so a captured call replays."""
    import torch
    import gpu_harness as H
    L = _lib.lib()
    split(0)
    w = WORKLOADS[1].scaled(B=1, H=33, S=2048)             # 264 row tiles: splits by itself, slots in the caller's workspace
    assert L.mi355_sage_attn_split_rule(w.B, w.H, w.S, w.S, w.D, 0) == 256
    q0, k0, v0 = (H.dev_bf16(x) for x in make_inputs(w))
    q, k, v = q0.clone(), k0.clone(), v0.clone()
    o = torch.empty_like(q)
    st = _lib.strides_bhnd(w.S, w.H, w.D)
    nws = L.mi355_sage_workspace_bytes(w.B, w.H, w.S, w.S, w.D, 0)
    ws = torch.empty(nws, dtype=torch.uint8, device="cuda")

    def call(out):
        rc = L.mi355_sage_sdpa_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), w.B, w.H, w.S, w.S, w.D,
                                    w.scale, st, st, st, st, 0, 0, 0, 0, 0, torch.cuda.current_stream().cuda_stream,
                                    0, ws.data_ptr(), nws)
        assert rc == 0, rc

    call(o)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(o)
    for rep in range(3):
        q.copy_(torch.roll(q0, rep, dims=1))
        k.copy_(k0 * (1.0 + 0.25 * rep))
        junk = (q.float() @ q.float().transpose(-1, -2)).sum()
        ws.fill_(0xAB)                                       # stale flags and slots must not matter
        torch.cuda.synchronize()
        o.zero_()
        g.replay()
        torch.cuda.synchronize()
        eager = torch.empty_like(o)
        call(eager)
        torch.cuda.synchronize()
        assert torch.isfinite(junk)
        np.testing.assert_array_equal(H.to_bits(o), H.to_bits(eager))


def test_the_e4m3_variant_keeps_one_workgroup_per_row_tile(split):
    """Its loop has no registers to spare for the hand-over: a forced split leaves its schedule, hence
    its bits, alone."""
    from test_gpu_attn import _one_shot
    w = WORKLOADS[4].scaled(B=2, H=3, S=700)
    q, k, v = make_inputs(w)
    split(-1)
    plain = _one_shot(q, k, v, w.scale, 1)
    split(64)
    np.testing.assert_array_equal(_one_shot(q, k, v, w.scale, 1), plain)


def test_split_mode_argument():
    L = _lib.lib()
    for bad in (-2, 12, 1032):
        assert L.mi355_sage_set_attn_split(bad) == -1
    assert L.mi355_sage_set_attn_split(0) == 0


def test_a_partial_result_that_never_arrives_poisons_rows_and_nothing_hangs(split):
    """The give-up path of the hand-over wait, forced from the host: in test mode no workgroup
    announces its partial result, every workgroup that needs one stops polling after 64 polls and
    writes NaN into its rows.  The launch ends, rows of items that were not cut stay right, and
    the next ordinary call is unaffected."""
    import torch
    import gpu_harness as H
    from test_gpu_attn import _one_shot
    L = _lib.lib()
    w = WORKLOADS[2].scaled(B=2, H=3, S=1100)               # 30 items of 18 steps; 24 workgroups: spans of 24 steps
    q, k, v = make_inputs(w)
    split(24)
    assert L.mi355_sage_attn_split_faults(1) >= 0           # (clears the device's count)
    good = bf16_bits_to_f32(_one_shot(q, k, v, w.scale, 0))
    assert L.mi355_sage_attn_split_faults(0) == 0           # a healthy run counts nothing
    assert L.mi355_sage_set_attn_split_wait(-64) == 0
    try:
        bad = bf16_bits_to_f32(_one_shot(q, k, v, w.scale, 0))
    finally:
        assert L.mi355_sage_set_attn_split_wait(0) == 0
    nan_rows = np.isnan(bad).any(axis=-1)                   # [B,S,H]
    assert nan_rows.any() and not nan_rows.all()
    # the device kept count of the workgroups that gave up: one per poisoned row tile of a head
    tiles = {(b, h, s // 256) for b, s, h in zip(*np.nonzero(nan_rows))}
    assert L.mi355_sage_attn_split_faults(0) == len(tiles)
    assert L.mi355_sage_attn_split_faults(1) == len(tiles) and L.mi355_sage_attn_split_faults(0) == 0
    # poisoned rows come as whole row tiles of a head; everything else is bit-identical
    np.testing.assert_array_equal(bad[~nan_rows], good[~nan_rows])
    assert np.isnan(bad[nan_rows]).all()
    again = bf16_bits_to_f32(_one_shot(q, k, v, w.scale, 0))
    np.testing.assert_array_equal(again, good)
    assert L.mi355_sage_attn_split_faults(0) == 0
    for bad_arg in (-(1 << 25), 1 << 25):
        assert L.mi355_sage_set_attn_split_wait(bad_arg) == -1
