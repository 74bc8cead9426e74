"""Quantized attention of the oracle (PARITY UNPINNED by reference data):
checked against the float64 numpy restatement on the same quantized tensors,
against the fp32 referee at the reference's own acceptance bars
(cosine >= 0.999, serenitymojo/parity.mojo:41), and through invariants."""
import numpy as np
import pytest
import torch

import np_restatement as R
from mojodiffusion_amd.workloads import WORKLOADS, make_inputs, bf16_bits_to_f32


def cos_maxabs(a, b):
    """serenitymojo/parity.mojo:57-93 (float64 cosine + max-abs)."""
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    den = np.sqrt((a * a).sum()) * np.sqrt((b * b).sum())
    cos = 1.0 if den == 0 else float((a * b).sum() / den)
    return cos, float(np.abs(a - b).max())


def _f16_codec(p):
    return p.astype(np.float16).astype(np.float32)


def _e4m3_codec_448(p):
    y = torch.from_numpy(np.ascontiguousarray(p * np.float32(448.0))).to(torch.float8_e4m3fn).to(torch.float32).numpy()
    return y / np.float32(448.0)


@pytest.mark.parametrize("wid,variant,mask", [(1, 0, (0, 0)), (2, 0, (0, 0)), (3, 0, (0, 0)), (4, 1, (0, 0)), (2, 1, (0, 0)),
                                              (2, 0, (30, 150)), (4, 1, (64, 128))])
def test_attn_matches_float64_restatement(oracle, wid, variant, mask):
    w = WORKLOADS[wid].scaled(B=1, H=2, S=200)     # ragged: 200 = 3*64 + 8
    q, k, v = make_inputs(w)
    mu, qmul, kmul = oracle.kstats(k, w.scale, 3, *mask)
    q8, qs = oracle.quant_q_ch(q, w.scale, qmul, w.blkq)
    k8, ks = oracle.quant_k_ch(k, mu, kmul, w.blkk, None, *mask)
    if variant == 0:
        vq, vs = oracle.quant_v_f16(v, w.blkk), None
        v_f32 = vq.view(np.float16).astype(np.float32)
        codec = _f16_codec
    else:
        vq, vs = oracle.quant_v_fp8(v, w.blkk, *mask)
        v_f32 = oracle.e4m3_to_f32(vq) * vs[:, :, None, :]
        codec = _e4m3_codec_448
    o16, o32 = oracle.attn(q8, qs, w.blkq, k8, ks, w.blkk, vq, vs, variant, w.S, w.S, *mask)
    want = R.attn_float64(q8, qs, w.blkq, k8, ks, w.blkk, v_f32, w.S, w.S, codec, variant == 1, *mask,
                          normalise_by_rounded=(variant == 1))
    # exp2f (libm) and np.exp2 may differ in the last ulp, which can flip one P rounding
    np.testing.assert_allclose(o32, want, atol=2e-4, rtol=1e-4)
    # bf16 epilogue is RNE of the fp32 value
    np.testing.assert_array_equal(o16, oracle.f32_to_bf16(o32))


@pytest.mark.parametrize("wid", [1, 2, 3, 4])
def test_whole_path_within_bars_of_fp32_referee(oracle, wid):
    w = WORKLOADS[wid].scaled(B=1, H=2, S=640)
    q, k, v = make_inputs(w)
    o16, o32 = oracle.sdpa_bf16(q, k, v, w.scale, variant=w.variant, blkq=w.blkq, blkk=w.blkk)
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k), bf16_bits_to_f32(v), w.scale)
    cos, mx = cos_maxabs(bf16_bits_to_f32(o16), ref)
    assert cos >= 0.999, (cos, mx)
    assert mx <= (4e-2 if w.variant == 0 else 6e-2), (cos, mx)


def test_balancing_is_what_carries_outlier_channels(oracle):
    """Workload 3 multiplies 1 % of the K channels by 8 (zero-mean outliers), which mean
    smoothing cannot remove: per-block INT8 alone lands below the 0.999 bar, the balanced
    recipe above it."""
    w = WORKLOADS[3].scaled(B=1, H=2, S=1100)
    q, k, v = make_inputs(w)
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k), bf16_bits_to_f32(v), w.scale)
    _, plain = oracle.sdpa_bf16(q, k, v, w.scale, blkq=w.blkq, blkk=w.blkk, balance=False)
    _, bal = oracle.sdpa_bf16(q, k, v, w.scale, blkq=w.blkq, blkk=w.blkk, balance=True)
    cos_plain, _ = cos_maxabs(plain, ref)
    cos_bal, mx = cos_maxabs(bal, ref)
    assert cos_plain < 0.999 <= 0.9995 <= cos_bal, (cos_plain, cos_bal)
    assert mx <= 4e-2, mx


@pytest.mark.parametrize("variant", [0, 1])
def test_key_range_mask_and_stats(oracle, variant):
    """Masking keys [lo, hi) equals attention over the remaining keys (same statistics, same
    blocks when the cut falls on block boundaries); Stats is the log-sum-exp of the scaled
    scores of the fp32 referee to quantization accuracy."""
    w = WORKLOADS[2].scaled(B=1, H=2, S=384)
    q, k, v = make_inputs(w)
    lo, hi = 128, 256
    o16, o32, st = oracle.sdpa_bf16(q, k, v, w.scale, variant=variant, blkq=128, blkk=64, mask_lo=lo, mask_hi=hi,
                                    want_stats=True)
    keep = np.r_[0:lo, hi:w.S]
    o16c, o32c, stc = oracle.sdpa_bf16(q, k[:, keep], v[:, keep], w.scale, variant=variant, blkq=128, blkk=64,
                                       want_stats=True)
    np.testing.assert_array_equal(o16, o16c)
    np.testing.assert_array_equal(st, stc)
    qf, kf, vf = (bf16_bits_to_f32(x) for x in (q, k, v))
    ref, lse = oracle.sdpa_f32(qf, kf, vf, w.scale, mask_lo=lo, mask_hi=hi, want_stats=True)
    refc = oracle.sdpa_f32(qf, kf[:, keep], vf[:, keep], w.scale)
    np.testing.assert_allclose(ref, refc, rtol=1e-6, atol=1e-7)
    cos, mx = cos_maxabs(o32, ref)
    assert cos >= 0.999, (cos, mx)
    np.testing.assert_allclose(st, lse, atol=3e-2)
    # float64 brute force of the referee's stats
    s = np.einsum("bihd,bjhd->bhij", qf.astype(np.float64), kf[:, keep].astype(np.float64)) * w.scale
    np.testing.assert_allclose(lse, np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1)) + s.max(-1), atol=1e-5)


def test_additive_mask(oracle):
    """An additive bias (serenitymojo/ops/attention.mojo:1596-1647): zeros change nothing, a
    -1e4 column block equals the key-range mask, a per-row constant cancels in the softmax."""
    w = WORKLOADS[2].scaled(B=1, H=2, S=192)
    q, k, v = make_inputs(w)
    qf, kf, vf = (bf16_bits_to_f32(x) for x in (q, k, v))
    zero = np.zeros((1, 2, w.S, w.S), np.float32)
    base = oracle.sdpa_f32(qf, kf, vf, w.scale)
    np.testing.assert_array_equal(oracle.sdpa_f32(qf, kf, vf, w.scale, addmask=zero), base)
    rng = np.random.default_rng(4)
    bias = rng.standard_normal((1, 2, w.S, w.S)).astype(np.float32)
    got = oracle.sdpa_f32(qf, kf, vf, w.scale, addmask=bias)
    s = np.einsum("bihd,bjhd->bhij", qf.astype(np.float64), kf.astype(np.float64)) * w.scale + bias
    p = np.exp(s - s.max(-1, keepdims=True))
    want = np.einsum("bhij,bjhd->bihd", p / p.sum(-1, keepdims=True), vf.astype(np.float64))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    block = zero.copy()
    block[..., 64:128] = -1e4
    np.testing.assert_allclose(oracle.sdpa_f32(qf, kf, vf, w.scale, addmask=block),
                               oracle.sdpa_f32(qf, kf, vf, w.scale, mask_lo=64, mask_hi=128), rtol=1e-6, atol=1e-7)
    # quantized path with the same bias stays within the bars of the biased referee
    _, o32 = oracle.sdpa_bf16(q, k, v, w.scale, addmask=bias)
    cos, mx = cos_maxabs(o32, got)
    assert cos >= 0.999 and mx <= 4e-2, (cos, mx)
    rowc = np.broadcast_to(rng.standard_normal((1, 2, w.S, 1)).astype(np.float32), zero.shape)
    _, o32c = oracle.sdpa_bf16(q, k, v, w.scale, addmask=rowc)
    _, o32z = oracle.sdpa_bf16(q, k, v, w.scale)
    np.testing.assert_allclose(o32c, o32z, atol=2e-3)


def test_e4m3_variant_returns_a_dominant_key_exactly(oracle):
    """One key far above the rest: the softmax is one-hot and O must be that key's V (to the
    precision of V's own e4m3 code), although the key's probability 2^(s - ceil(s)) is not an
    e4m3 number — the normaliser sums the rounded probabilities."""
    w = WORKLOADS[2].scaled(B=1, H=1, S=128, k_offset_std=0.0)
    q, k, v = make_inputs(w)
    kf = bf16_bits_to_f32(k)
    kf[:, 77] = bf16_bits_to_f32(q)[:, 5] * 6.0          # aligned with query 5: score ~ 6*|q|^2*scale
    from mojodiffusion_amd.workloads import f32_to_bf16_bits
    _, o32 = oracle.sdpa_bf16(q, f32_to_bf16_bits(kf), v, w.scale, variant=1, blkq=32, blkk=64)
    v8, vs = oracle.quant_v_fp8(v, 64)
    v_deq = oracle.e4m3_to_f32(v8)[0, 0, 77] * vs[0, 0]
    np.testing.assert_allclose(o32[0, 5, 0], v_deq, rtol=1e-5, atol=1e-6)


def test_k_smoothing_rescues_offset_keys(oracle):
    """With a large per-channel K offset, un-smoothed INT8 K loses the signal;
    smoothed K keeps the fp32 answer (softmax is invariant to the removed mean)."""
    w = WORKLOADS[2].scaled(B=1, H=2, S=384, k_offset_std=16.0)
    q, k, v = make_inputs(w)
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k), bf16_bits_to_f32(v), w.scale)
    _, o_s = oracle.sdpa_bf16(q, k, v, w.scale, smooth_k=True)
    _, o_n = oracle.sdpa_bf16(q, k, v, w.scale, smooth_k=False)
    cos_s, _ = cos_maxabs(o_s, ref)
    cos_n, _ = cos_maxabs(o_n, ref)
    assert cos_s >= 0.999 and cos_s > cos_n


def test_rectangular_and_row_subset(oracle):
    """Query rows are independent: a whole-block slice of Q against the full K/V
    reproduces those rows bit-for-bit."""
    w = WORKLOADS[2].scaled(B=1, H=2, S=512)
    q, k, v = make_inputs(w)
    full16, _ = oracle.sdpa_bf16(q, k, v, w.scale)
    part16, _ = oracle.sdpa_bf16(q[:, 128:256], k, v, w.scale)
    np.testing.assert_array_equal(part16, full16[:, 128:256])


def test_constant_v_and_single_key(oracle):
    w = WORKLOADS[1].scaled(B=1, H=1, S=64)
    q, k, v = make_inputs(w)
    v[:] = v[:, :1]                                  # constant V rows -> O = V (up to P rounding)
    o16, o32 = oracle.sdpa_bf16(q, k, v, w.scale, blkq=64, blkk=64)
    np.testing.assert_allclose(o32, np.broadcast_to(bf16_bits_to_f32(v[:, :1]), o32.shape), atol=2e-3)
    # one key: softmax is 1, O = fp16(V) exactly
    o16, o32 = oracle.sdpa_bf16(q, k[:, :1], v[:, :1], w.scale, blkq=64, blkk=64)
    np.testing.assert_array_equal(o32, np.broadcast_to(bf16_bits_to_f32(v[:, :1]), o32.shape))
