"""GPU parity of the quantize kernels, through the C ABI, against the CPU
checker: INT8 codes, fp32 scales, the K statistics (mean, channel multipliers),
fp16 / e4m3 V and V scales must be bit-identical."""
import ctypes

import numpy as np
import pytest

from mojodiffusion_amd import _lib
from mojodiffusion_amd.workloads import WORKLOADS, make_inputs, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def _check_qk(oracle, H, q, k, scale, blkq, blkk, smooth, balance=True, mask=(0, 0)):
    g = H.quant_qk(q, k, scale, blkq, blkk, smooth, balance=balance, mask=mask)
    want = H.oracle_quant_qk(oracle, q, k, scale, blkq, blkk, smooth, balance, mask)
    q8, qs, k8, ks = want["q8"], want["qscale"], want["k8"], want["kscale"]
    for name in ("kmean", "qmul", "kmul"):
        np.testing.assert_array_equal(g[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    nqb, nkb = qs.shape[2], ks.shape[2]
    np.testing.assert_array_equal(g["qscale"][:, :, :nqb].view(np.uint32), qs.view(np.uint32))
    np.testing.assert_array_equal(g["kscale"][:, :, :nkb].view(np.uint32), ks.view(np.uint32))
    assert np.all(g["qscale"][:, :, nqb:] == 1.0) and np.all(g["kscale"][:, :, nkb:] == 1.0)
    np.testing.assert_array_equal(g["q8"], q8)           # includes the zero pad rows
    np.testing.assert_array_equal(g["k8"], k8)
    return g


@pytest.mark.parametrize("wid", [1, 2, 3, 4])
def test_quant_qk_bit_exact_workload_stats(oracle, wid):
    import gpu_harness as H
    w = WORKLOADS[wid]
    w = w if wid == 1 else w.scaled(B=w.B, H=3, S=1100)      # ragged: 1100 = 8*128 + 76 = 17*64 + 12
    q, k, _ = make_inputs(w)
    _check_qk(oracle, H, q, k, w.scale, w.blkq, w.blkk, True)
    _check_qk(oracle, H, q, k, w.scale, w.blkq, w.blkk, True, balance=False)


@pytest.mark.parametrize("wid", [2, 3, 4, 5])
def test_quant_bit_exact_at_full_sequence_length(oracle, wid):
    """Every workload at its real sequence length (c5: S = 32760 = 511*64 + 56, a ragged last
    block in every tensor) on two heads: statistics, INT8 codes and scales of Q and K, and for
    the e4m3 workloads the V bytes and scales, bit for bit."""
    import gpu_harness as H
    w = WORKLOADS[wid].scaled(B=1, H=2)
    q, k, v = make_inputs(w)
    _check_qk(oracle, H, q, k, w.scale, w.blkq, w.blkk, True)
    g = H.quant_v(v, w.variant)
    if w.variant == 0:
        np.testing.assert_array_equal(H.untile_v(g["vq"], 0), oracle.quant_v_f16(v, 128))
    else:
        v8, vs = oracle.quant_v_fp8(v, 128)
        np.testing.assert_array_equal(g["vscale"].view(np.uint32), vs.view(np.uint32))
        np.testing.assert_array_equal(H.untile_v(g["vq"], 1), v8)


@pytest.mark.parametrize("D,S,mask,smooth,balance", [(128, 700, (300, 512), True, True), (128, 333, (0, 64), True, True),
                                                     (64, 520, (500, 520), True, False), (128, 200, (17, 150), False, True),
                                                     (256, 600, (100, 333), True, True)])
def test_quant_with_masked_key_range(oracle, D, S, mask, smooth, balance):
    """Keys [lo, hi) take no part: not in the K statistics, not in their scale blocks (code 0),
    not in the V scales (bytes 0) — also when the range cuts through blocks and groups."""
    import gpu_harness as H
    rng = np.random.default_rng(S + D)
    q = f32_to_bf16_bits(rng.standard_normal((2, S, 2, D)).astype(np.float32))
    kx = (rng.standard_normal((2, S, 2, D)) * 2 + rng.standard_normal((2, 1, 2, D)) * 3).astype(np.float32)
    vx = rng.standard_normal((2, S, 2, D)).astype(np.float32)
    kx[:, mask[0]:mask[1]] *= 50.0                       # would dominate every statistic if it counted
    vx[:, mask[0]:mask[1]] *= 50.0
    k, v = f32_to_bf16_bits(kx), f32_to_bf16_bits(vx)
    g = _check_qk(oracle, H, q, k, 0.09, 128, 64, smooth, balance, mask)
    assert not g["k8"][:, :, mask[0]:mask[1]].any()
    g0 = H.quant_v(v, 0, mask)
    np.testing.assert_array_equal(H.untile_v(g0["vq"], 0), oracle.quant_v_f16(v, 128, *mask))
    g1 = H.quant_v(v, 1, mask)
    v8, vs = oracle.quant_v_fp8(v, 128, *mask)
    np.testing.assert_array_equal(g1["vscale"].view(np.uint32), vs.view(np.uint32))
    np.testing.assert_array_equal(H.untile_v(g1["vq"], 1), v8)


@pytest.mark.parametrize("D,blkq,blkk,S,smooth", [
    (64, 32, 32, 96, True), (64, 128, 128, 300, False), (128, 32, 64, 1, True),
    (128, 64, 32, 65, True), (128, 128, 64, 257, False), (64, 64, 64, 1024, True),
    (256, 128, 64, 1153, True), (256, 32, 32, 300, True), (256, 64, 128, 77, False)])
def test_quant_qk_bit_exact_shapes(oracle, D, blkq, blkk, S, smooth):
    import gpu_harness as H
    rng = np.random.default_rng(S * 7 + D)
    q = f32_to_bf16_bits(rng.standard_normal((2, S, 2, D)).astype(np.float32))
    k = f32_to_bf16_bits((rng.standard_normal((2, S, 2, D)) * 3 + rng.standard_normal((2, 1, 2, D)) * 5).astype(np.float32))
    _check_qk(oracle, H, q, k, 0.2, blkq, blkk, smooth)
    _check_qk(oracle, H, q, k, 0.2, blkq, blkk, smooth, balance=False)


def test_quant_qk_ties_zero_blocks_and_extremes(oracle):
    """Adversarial inputs: exact .5 ties (absmax 127 -> scale 1), an all-zero
    block, subnormal-scale blocks and bf16 extremes."""
    import gpu_harness as H
    D, S = 64, 256
    x = np.zeros((1, S, 1, D), np.float32)
    ties = np.float32([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, 64.5, -126.5, 126.5, 0.25, 0.75, -0.75])
    x[0, 0, 0, :len(ties)] = ties                         # block 0: ties
    # block 1 (rows 64..127): all zero
    x[0, 128:192] = np.random.default_rng(5).standard_normal((64, 1, D)) * 1e-30      # block 2: tiny values
    x[0, 192:256] = np.random.default_rng(6).standard_normal((64, 1, D)) * 1e30       # block 3: huge values
    k = f32_to_bf16_bits(x)
    q = f32_to_bf16_bits(np.random.default_rng(7).standard_normal((1, S, 1, D)).astype(np.float32))
    g = _check_qk(oracle, H, q, k, 1.0, 64, 64, False, balance=False)
    # balanced, with a spread the channel factors can carry without leaving the normal fp32 range
    # (values below 2^-126 are where a GPU that flushes subnormals and the CPU stop agreeing)
    x[0, 128:192] *= 1e18
    x[0, 192:256] *= 1e-18
    _check_qk(oracle, H, q, f32_to_bf16_bits(x), 1.0, 64, 64, False)
    assert g["kscale"][0, 0, 0] == 1.0 and g["kscale"][0, 0, 1] == 1.0
    np.testing.assert_array_equal(g["k8"][0, 0, 0, :len(ties)],
                                  np.int8([127, 0, 2, 2, 0, -2, -2, 64, 64, -126, 126, 0, 1, -1]))


def test_quant_qk_bhsd_strides_and_offsets(oracle):
    """The same logical tensor presented head-major ([B,H,S,D] memory) and at a
    non-zero element offset inside a larger buffer gives identical codes."""
    import gpu_harness as H
    rng = np.random.default_rng(21)
    B, S, Hh, D = 2, 200, 3, 128
    q = f32_to_bf16_bits(rng.standard_normal((B, S, Hh, D)).astype(np.float32))
    k = f32_to_bf16_bits(rng.standard_normal((B, S, Hh, D)).astype(np.float32) + 2.0)
    ref = H.quant_qk(q, k, 0.1, 128, 64, True)
    off = 64
    def bhsd_buf(x):
        flat = np.zeros(off + x.size, np.uint16)
        flat[off:] = np.ascontiguousarray(x.transpose(0, 2, 1, 3)).reshape(-1)
        return flat
    st = (ctypes.c_int64 * 4)(Hh * S * D, S * D, D, 1)
    got = H.quant_qk(bhsd_buf(q), bhsd_buf(k), 0.1, 128, 64, True, strides_q=st, strides_k=st,
                     q_off=off, k_off=off, shape=(B, Hh, S, S, D))
    for name in ("q8", "qscale", "k8", "kscale", "kmean", "qmul", "kmul"):
        np.testing.assert_array_equal(got[name], ref[name])
    # V presented the same way: BHSD memory at a non-zero offset
    v = f32_to_bf16_bits(rng.standard_normal((B, S, Hh, D)).astype(np.float32) * 2.0)
    for variant in (0, 1):
        a = H.quant_v(v, variant)
        b = H.quant_v(bhsd_buf(v), variant, strides=st, v_off=off, shape=(B, Hh, S, D))
        np.testing.assert_array_equal(a["vq"], b["vq"])
        if variant == 1:
            np.testing.assert_array_equal(a["vscale"], b["vscale"])


@pytest.mark.parametrize("D,S", [(128, 1100), (64, 1024), (128, 64), (64, 7), (256, 1153), (256, 50)])
def test_quant_v_bit_exact(oracle, D, S):
    import gpu_harness as H
    rng = np.random.default_rng(S + D)
    x = rng.standard_normal((2, S, 3, D)).astype(np.float32) * np.exp(rng.uniform(-3, 3, (1, 1, 3, D))).astype(np.float32)
    x[:, :, 1, 5] = 0.0                                    # all-zero channel -> scale 1.0
    if S > 10:
        x[0, 3, 0, 0] = 1e6                                # beyond fp16 range: saturates
    v = f32_to_bf16_bits(x)
    g0 = H.quant_v(v, 0)
    np.testing.assert_array_equal(H.untile_v(g0["vq"], 0), oracle.quant_v_f16(v, 128))
    g1 = H.quant_v(v, 1)
    v8, vs = oracle.quant_v_fp8(v, 128)
    np.testing.assert_array_equal(g1["vscale"].view(np.uint32), vs.view(np.uint32))
    np.testing.assert_array_equal(H.untile_v(g1["vq"], 1), v8)


def test_quant_v_fp8_every_bf16_value_and_rounding_tie(oracle):
    """Channels whose largest magnitude is 448 have the scale 1.0, so the quotient is the input
    itself: every bf16 value from 2^-13 to 448 of either sign goes through, among them every exact
    tie between two e4m3 codes (normal and subnormal range), both zeros, and values that round to
    zero.  Other channels repeat the values under scales 1.5, 3 and 1/3 (quotients that need the
    correction step of the division)."""
    import gpu_harness as H
    bits = np.arange(0x3900, 0x43E1, dtype=np.uint16)                 # 2^-13 .. 448
    vals = np.concatenate([bits, bits | 0x8000, np.uint16([0x0000, 0x8000])])
    D, Hh = 128, 1
    S = 64 * ((len(vals) + 1 + 63) // 64)
    v = np.zeros((1, S, Hh, D), np.uint16)
    for c in range(D):
        top = np.float32([448.0, 448.0 * 1.5, 448.0 * 3.0, 448.0 / 3.0][c % 4])
        col = np.roll(vals, 37 * c)
        if c % 4:                                                       # scaled copies: value * scale, rounded to bf16
            f = (col.astype(np.uint32) << 16).view(np.float32) * np.float32([1.0, 1.5, 3.0, 1.0 / 3.0][c % 4])
            col = f32_to_bf16_bits(f.reshape(1, -1, 1, 1)).reshape(-1)
            col = np.where((col & 0x7FFF) > f32_to_bf16_bits(np.float32([[[[top]]]])).reshape(-1)[0], np.uint16(0), col)
        v[0, :len(col), 0, c] = col
        v[0, len(vals), 0, c] = f32_to_bf16_bits(np.float32([[[[top]]]])).reshape(-1)[0]
    g = H.quant_v(v, 1)
    v8, vs = oracle.quant_v_fp8(v, 128)
    assert vs[0, 0, 0] == 1.0
    np.testing.assert_array_equal(g["vscale"].view(np.uint32), vs.view(np.uint32))
    np.testing.assert_array_equal(H.untile_v(g["vq"], 1), v8)


def test_quant_non_finite_inputs_follow_the_plain_formulas(oracle):
    """An infinity or a NaN among the inputs: the kernels' short cuts (reciprocal instead of divide,
    rounding by a magic addend, the conversion instruction) mean nothing then, and a wave that sees
    one takes the plain formulas — the codes and scales are still the checker's."""
    import gpu_harness as H
    rng = np.random.default_rng(77)
    B, S, Hh, D = 1, 256, 2, 128
    def tensor():
        return rng.standard_normal((B, S, Hh, D)).astype(np.float32)
    q, k, v = tensor(), tensor(), tensor()
    q[0, 5, 0, 17] = np.nan
    k[0, 70, 1, 3] = np.nan
    v[0, 9, 0, 100] = np.nan
    v[0, 200, 1, 64] = np.inf
    qb, kb, vb = f32_to_bf16_bits(q), f32_to_bf16_bits(k), f32_to_bf16_bits(v)
    g = H.quant_qk(qb, kb, 0.1, 128, 64, False, balance=False)
    want = H.oracle_quant_qk(oracle, qb, kb, 0.1, 128, 64, False, False, (0, 0))
    np.testing.assert_array_equal(g["q8"][:, :, :S], want["q8"][:, :, :S])
    np.testing.assert_array_equal(g["k8"][:, :, :S], want["k8"][:, :, :S])
    np.testing.assert_array_equal(g["qscale"][:, :, :S // 128].view(np.uint32), want["qscale"].view(np.uint32))
    g1 = H.quant_v(vb, 1)
    v8, vs = oracle.quant_v_fp8(vb, 128)
    np.testing.assert_array_equal(g1["vscale"].view(np.uint32), vs.view(np.uint32))
    np.testing.assert_array_equal(H.untile_v(g1["vq"], 1), v8)


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("wid,S,mask", [(2, 1100, (0, 0)), (1, 520, (0, 0)), (4, 700, (130, 260))])
def test_three_launch_stage_equals_the_separate_stages(wid, S, mask, variant):
    """mi355_sage_quant_qkv_bf16 runs the quantizers the way the one-shot calls do (three launches with
    shared roles); its outputs are those of the Q/K and V stage entry points, which the tests above
    hold to the CPU checker, bit for bit."""
    import gpu_harness as H
    w = WORKLOADS[wid].scaled(B=2, H=3, S=S)
    q, k, v = make_inputs(w)
    blkq = 128 if variant == 0 else 32
    got = H.quant_qkv(q, k, v, w.scale, variant, blkq, 64, mask=mask)
    qk = H.quant_qk(q, k, w.scale, blkq, 64, True, mask=mask)
    vv = H.quant_v(v, variant, mask=mask)
    for name in ("q8", "k8"):
        np.testing.assert_array_equal(got[name], qk[name], err_msg=name)
    for name in ("qscale", "kscale", "kmean", "qmul", "kmul"):
        np.testing.assert_array_equal(got[name].view(np.uint32), qk[name].view(np.uint32), err_msg=name)
    np.testing.assert_array_equal(got["vq"], vv["vq"])
    if variant == 1:
        np.testing.assert_array_equal(got["vscale"].view(np.uint32), vv["vscale"].view(np.uint32))
    # without the Q encode (q8 == qscale == NULL): everything else as before, the Q outputs untouched
    rest = H.quant_qkv(q, k, v, w.scale, variant, blkq, 64, mask=mask, encode_q=False)
    for name in ("k8", "kscale", "kmean", "qmul", "kmul", "vq"):
        np.testing.assert_array_equal(rest[name], got[name], err_msg=name)
    assert np.all(rest["q8"] == 77) and np.all(rest["qscale"] == -1.0)


def test_quant_full_size_properties():
    """Workload 2 at full size: size-independent properties of the device output
    (no CPU pass over 14 M elements per tensor needed)."""
    import torch
    import gpu_harness as H
    w = WORKLOADS[2]
    q, k, _ = make_inputs(w)
    g = H.quant_qk(q, k, w.scale, w.blkq, w.blkk, True, balance=False)
    q8, k8 = g["q8"].astype(np.int32), g["k8"].astype(np.int32)
    # every block's absmax code is exactly 127 and -128 never appears
    assert np.all(np.abs(q8).reshape(w.B, w.H, -1, w.blkq * w.D).max(-1) == 127)
    assert np.all(np.abs(k8).reshape(w.B, w.H, -1, w.blkk * w.D).max(-1) == 127)
    assert q8.min() >= -127 and k8.min() >= -127
    # dequantised K + mean reproduces K within half a step per element
    kf = (k.astype(np.uint32) << 16).view(np.float32).transpose(0, 2, 1, 3)
    deq = k8 * np.repeat(g["kscale"], w.blkk, axis=2)[..., None] + g["kmean"][:, :, None, :]
    step = np.repeat(g["kscale"], w.blkk, axis=2)[..., None]
    assert np.all(np.abs(deq - kf) <= 0.5 * step * (1 + 1e-5) + 1e-6)
    # the mean is the column mean
    np.testing.assert_allclose(g["kmean"], kf.astype(np.float64).mean(2), rtol=0, atol=1e-6)
