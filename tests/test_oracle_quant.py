"""The quantizers have no counterpart in the reference (PARITY UNPINNED by
reference data); these tests pin the C oracle with closed forms, invariants and
the independent numpy restatement in np_restatement.py."""
import numpy as np
import pytest

import np_restatement as R
from mojodiffusion_amd.workloads import WORKLOADS, make_inputs, f32_to_bf16_bits


def _rand_bits(rng, shape, std=1.0):
    return f32_to_bf16_bits(rng.standard_normal(shape).astype(np.float32) * np.float32(std))


@pytest.mark.parametrize("S,blkq,mult", [(256, 64, 64), (200, 128, 128), (77, 32, 128), (130, 64, 64)])
def test_quant_q_matches_numpy(oracle, S, blkq, mult):
    rng = np.random.default_rng(S)
    q = _rand_bits(rng, (2, S, 3, 64))
    scale = 0.125
    q8, qs = oracle.quant_q(q, scale, blkq, mult)
    q8n, qsn = R.quant_q(q, scale, blkq, mult)
    np.testing.assert_array_equal(qs, qsn)
    np.testing.assert_array_equal(q8, q8n)


def test_quant_closed_forms(oracle):
    rng = np.random.default_rng(11)
    B, S, H, D, blk = 1, 192, 2, 32, 64
    k = _rand_bits(rng, (B, S, H, D))
    k[:, 64:128, 1, :] = 0                       # an all-zero block
    k8, ks = oracle.quant_k(k, None, blk)
    x = R.bf16_to_f32(k).transpose(0, 2, 1, 3)
    assert ks[0, 1, 1] == 1.0 and not k8[0, 1, 64:128].any()
    for h in range(H):
        for t in range(S // blk):
            tile = x[0, h, t * blk:(t + 1) * blk]
            codes = k8[0, h, t * blk:(t + 1) * blk].astype(np.int32)
            if not tile.any():
                continue
            i = np.unravel_index(np.abs(tile).argmax(), tile.shape)
            assert abs(codes[i]) == 127                      # the absmax element maps to +-127
            assert codes.min() >= -127 and codes.max() <= 127  # -128 is never produced
            err = np.abs(tile.astype(np.float64) / np.float64(ks[0, h, t]) - codes)
            assert err.max() <= 0.5 + 1e-5              # + one fp32 rounding of x/scale (|x/scale| <= 127)
            assert np.float32(ks[0, h, t]) == np.float32(np.abs(tile).max()) / np.float32(127.0)


def test_quant_ties_to_even(oracle):
    """A block whose absmax is exactly 127 has scale 1, so x = n + 0.5 are exact ties."""
    D = 32
    vals = np.float32([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, 64.5, -126.5, 126.5, 0.25, 0.75, -0.75])
    x = np.zeros((1, 64, 1, D), np.float32)
    x[0, 0, 0, :len(vals)] = vals
    k8, ks = oracle.quant_k(f32_to_bf16_bits(x), None, 64)
    assert ks[0, 0, 0] == 1.0
    want = np.int8([127, 0, 2, 2, 0, -2, -2, 64, 64, -126, 126, 0, 1, -1])
    np.testing.assert_array_equal(k8[0, 0, 0, :len(vals)], want)


@pytest.mark.parametrize("S", [64, 100, 1000])
def test_kmean_exact_and_blocked(oracle, S):
    rng = np.random.default_rng(S)
    k = f32_to_bf16_bits(rng.standard_normal((2, S, 2, 16)).astype(np.float32)
                         + 3.0 * rng.standard_normal((2, 1, 2, 16)).astype(np.float32))
    mu = oracle.kmean(k)
    np.testing.assert_array_equal(mu, R.kmean_blocked(k))
    np.testing.assert_array_equal(mu, R.kmean_exact(k))     # exact whenever the fp64 sums are exact


def test_kmean_order_is_the_blocked_one(oracle):
    """With a magnitude spread beyond 2^53 the order matters; the oracle must
    follow the leaf/group tree, not a straight running sum."""
    S, D = 48, 1
    x = np.zeros((1, S, 1, D), np.float32)
    x[0, 0] = 2.0 ** 60
    x[0, 1:16] = 1.0                                  # leaf 0: absorbed by 2^60
    x[0, 16] = -(2.0 ** 60)
    x[0, 17:48] = 1.0                                 # leaf 1: absorbed; leaf 2: 16 survives
    mu = oracle.kmean(f32_to_bf16_bits(x))
    np.testing.assert_array_equal(mu, R.kmean_blocked(f32_to_bf16_bits(x)))
    assert mu[0, 0, 0] == np.float32(16.0 / S)


@pytest.mark.parametrize("wid", [1, 2, 3])
def test_quant_k_smoothed_matches_numpy_on_workload_stats(oracle, wid):
    w = WORKLOADS[wid].scaled(B=1, H=2, S=320)
    _, k, _ = make_inputs(w)
    mu = oracle.kmean(k)
    k8, ks = oracle.quant_k(k, mu, w.blkk)
    k8n, ksn = R.quant_k(k, R.kmean_blocked(k), w.blkk, w.blkk)
    np.testing.assert_array_equal(ks, ksn)
    np.testing.assert_array_equal(k8, k8n)
    if w.k_offset_std > 0:
        # smoothing must shrink the scales when K carries a per-channel offset
        _, ks_raw = oracle.quant_k(k, None, w.blkk)
        assert ks.mean() < 0.6 * ks_raw.mean()


@pytest.mark.parametrize("smooth,balance", [(True, True), (False, True), (True, False), (False, False)])
@pytest.mark.parametrize("S,mask", [(320, (0, 0)), (300, (40, 200)), (130, (64, 128)), (200, (150, 200))])
def test_kstats_and_balanced_quantizers_match_numpy(oracle, smooth, balance, S, mask):
    """Per-channel statistics (mean, balancing factor) and the Q / K codes they lead to, against
    the numpy restatement (exact mean by math.fsum, numpy's correctly rounded sqrt and divide)."""
    w = WORKLOADS[3].scaled(B=1, H=2, S=S)               # two K channels of each head carry 8x the range
    q, k, _ = make_inputs(w)
    flags = (1 if smooth else 0) | (2 if balance else 0)
    mu, qmul, kmul = oracle.kstats(k, w.scale, flags, *mask)
    mu_n, qmul_n, kmul_n = R.kstats(k, w.scale, smooth, balance, *mask)
    np.testing.assert_array_equal(mu, mu_n)
    np.testing.assert_array_equal(qmul, qmul_n)
    np.testing.assert_array_equal(kmul, kmul_n)
    k8, ks = oracle.quant_k_ch(k, mu, kmul, w.blkk, 128, *mask)
    k8n, ksn = R.quant_k(k, mu_n, w.blkk, 128, kmul_n, *mask)
    np.testing.assert_array_equal(ks, ksn)
    np.testing.assert_array_equal(k8, k8n)
    q8, qs = oracle.quant_q_ch(q, w.scale, qmul, w.blkq, 256)
    q8n, qsn = R.quant_q_ch(q, qmul_n, w.blkq, 256)
    np.testing.assert_array_equal(qs, qsn)
    np.testing.assert_array_equal(q8, q8n)
    if mask[1] > mask[0]:
        assert not k8[:, :, mask[0]:mask[1]].any()       # masked keys carry code 0


def test_kstats_closed_forms(oracle):
    """What the balancing factor is, independent of any restatement: s_d^2 is the channel's
    largest |k - mean|; qmul * kmul is c up to the two roundings; with both flags clear the
    multipliers are exactly (c, 1) and the mean 0; the balanced channels all have the same
    largest magnitude sqrt(amax) on the K side; and the scores q.k are unchanged."""
    w = WORKLOADS[3].scaled(B=1, H=2, S=256)
    q, k, _ = make_inputs(w)
    c = np.float32(np.float64(np.float32(w.scale)) * R.LOG2E)
    mu0, qm0, km0 = oracle.kstats(k, w.scale, 0)
    assert not mu0.any() and np.all(qm0 == c) and np.all(km0 == 1.0)
    mu, qm, km = oracle.kstats(k, w.scale, 3)
    x = R.bf16_to_f32(k).transpose(0, 2, 1, 3)
    amax = np.abs((x - mu[:, :, None, :]).astype(np.float32)).max(axis=2)
    sd = qm / c
    np.testing.assert_allclose(sd.astype(np.float64) ** 2, amax, rtol=3e-7)
    np.testing.assert_allclose(qm.astype(np.float64) * km, c, rtol=2e-7)
    # the two outlier channels of each head get a factor ~sqrt(8) above the rest
    ratio = np.sort(sd, axis=-1)
    assert np.all(ratio[..., -2] > 2.0 * ratio[..., -3]) and np.all(ratio[..., -3] < 1.5 * ratio[..., 0])
    kb = ((x - mu[:, :, None, :]).astype(np.float32) * km[:, :, None, :]).astype(np.float32)
    np.testing.assert_allclose(np.abs(kb).max(axis=2), np.sqrt(amax), rtol=3e-7)
    qb = R.bf16_to_f32(q).transpose(0, 2, 1, 3) * qm[:, :, None, :]
    s_bal = np.einsum("bhid,bhjd->bhij", qb.astype(np.float64), kb.astype(np.float64))
    s_raw = np.einsum("bhid,bhjd->bhij", (R.bf16_to_f32(q).transpose(0, 2, 1, 3) * c).astype(np.float64),
                      (x - mu[:, :, None, :]).astype(np.float64))
    np.testing.assert_allclose(s_bal, s_raw, atol=2e-5)
    # a constant channel has nothing to balance: factor 1
    k2 = k.copy()
    k2[:, :, 0, 7] = k2[0, 0, 0, 7]
    _, qm2, km2 = oracle.kstats(k2, w.scale, 3)
    assert np.all(km2[:, 0, 7] == 1.0) and np.all(qm2[:, 0, 7] == c)
    # masked keys do not influence the statistics
    k3 = k.copy()
    k3[:, 100:180] = f32_to_bf16_bits(np.full((1, 80, 2, w.D), 1000.0, np.float32))
    a = oracle.kstats(k, w.scale, 3, 100, 180)
    b = oracle.kstats(k3, w.scale, 3, 100, 180)
    for u, v in zip(a, b):
        np.testing.assert_array_equal(u, v)
    assert oracle.lib().sage_oracle_kstats(None, 1, 1, 1, 1, None, 1.0, 0, 0, 0, None, None, None) == -1


def test_quant_v(oracle):
    rng = np.random.default_rng(13)
    v = _rand_bits(rng, (2, 150, 3, 32), std=3.0)
    v[:, :, 1, 5] = 0                                  # all-zero channel -> scale 1.0
    v16 = oracle.quant_v_f16(v, 64)
    np.testing.assert_array_equal(v16, R.quant_v_f16(v, 64))
    v8, vs = oracle.quant_v_fp8(v, 64)
    v8n, vsn = R.quant_v_fp8(v, 64)
    np.testing.assert_array_equal(vs, vsn)
    np.testing.assert_array_equal(v8, v8n)
    assert np.all(vs[:, 1, 5] == 1.0)
    # the channel absmax maps to +-448 exactly
    dec = oracle.e4m3_to_f32(v8)
    assert np.all(np.abs(dec[:, :, :150]).max(axis=2)[vs != 1.0] == 448.0)
    # channel maximum over the kept keys only; masked rows stay 0
    v[:, 20:40] = f32_to_bf16_bits(np.full((2, 20, 3, 32), 50.0, np.float32))
    v8m, vsm = oracle.quant_v_fp8(v, 64, 20, 40)
    v8mn, vsmn = R.quant_v_fp8(v, 64, 20, 40)
    np.testing.assert_array_equal(vsm, vsmn)
    np.testing.assert_array_equal(v8m, v8mn)
    np.testing.assert_array_equal(vsm, oracle.quant_v_fp8(np.delete(v, np.s_[20:40], axis=1), 64)[1])
    assert not v8m[:, :, 20:40].any()
    v16m = oracle.quant_v_f16(v, 64, 20, 40)
    np.testing.assert_array_equal(v16m, R.quant_v_f16(v, 64, 20, 40))
    assert not v16m[:, :, 20:40].any() and v16m[:, :, :20].any()


def test_bad_args(oracle):
    L = oracle.lib()
    q = np.zeros((1, 8, 1, 8), np.uint16)
    import ctypes
    p = q.ctypes.data_as(ctypes.c_void_p)
    st = oracle.strides_bshd(8, 1, 8)
    out = np.zeros(64, np.int8).ctypes.data_as(ctypes.c_void_p)
    sc = np.zeros(4, np.float32).ctypes.data_as(ctypes.c_void_p)
    assert L.sage_oracle_quant_q(None, 1, 1, 8, 8, st, 1.0, 8, 8, out, sc) == -1
    assert L.sage_oracle_quant_q(p, 1, 1, 0, 8, st, 1.0, 8, 8, out, sc) == -1
    assert L.sage_oracle_quant_q(p, 1, 1, 8, 8, st, 1.0, 0, 8, out, sc) == -1
