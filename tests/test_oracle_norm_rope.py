"""The two ops in front of the path (RMSNorm over the head dim, interleaved RoPE) as the CPU
checker restates them, against the vectors the reference's own smoke tests hold, the closed
form its large-D test uses, algebraic properties, and an independent numpy restatement."""
import json
import os

import numpy as np
import pytest

import np_restatement as R
from mojodiffusion_amd.workloads import f32_to_bf16_bits, bf16_bits_to_f32

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def kat():
    with open(os.path.join(HERE, "golden", "ops_smoke_rmsnorm_rope_kat.json")) as f:
        return json.load(f)


def test_rms_norm_reference_vector(oracle, kat):
    """serenitymojo/ops_smoke.mojo:78-96."""
    x = np.array(kat["rms_x"], np.float32).reshape(3, 6)
    g = np.array(kat["rms_g"], np.float32)
    got = oracle.rms_norm_f32(x, g, kat["rms_eps"])
    np.testing.assert_allclose(got, np.array(kat["rms_y"]).reshape(3, 6), rtol=0, atol=2e-7)


def test_rope_reference_vector(oracle, kat):
    """serenitymojo/ops_smoke2.mojo:92-120."""
    x = np.array(kat["rope_x"], np.float32).reshape(3, 8)
    c = np.array(kat["rope_cos"], np.float32).reshape(3, 4)
    s = np.array(kat["rope_sin"], np.float32).reshape(3, 4)
    got = oracle.rope_interleaved_f32(x, c, s)
    np.testing.assert_allclose(got, np.array(kat["rope_y_interleaved"]).reshape(3, 8), rtol=0, atol=3e-7)
    # the same inputs in the half-split pairing (x[i], x[i + D/2]): y_half_ref of the same test
    got = oracle.rope_halfsplit_f32(x, c, s)
    np.testing.assert_allclose(got, np.array(kat["rope_y_halfsplit"]).reshape(3, 8), rtol=0, atol=3e-7)
    # the two pairings are one rotation seen through a permutation of the channels
    perm = np.concatenate([np.arange(0, 8, 2), np.arange(1, 8, 2)])          # interleaved -> half-split order
    np.testing.assert_array_equal(oracle.rope_interleaved_f32(x, c, s)[:, perm], oracle.rope_halfsplit_f32(x[:, perm], c, s))


@pytest.mark.parametrize("D", [64, 128, 2560, 3072, 4096])
def test_rms_norm_closed_form_at_scale(oracle, D):
    """The sequence and float64 closed form of serenitymojo/ops_smoke2.mojo:372-403 (there for
    D = 2560, 3072, 4096; the head dims 64 and 128 of this path added)."""
    i = np.arange(D)
    x = (np.float32(0.5) + (i % 17).astype(np.float32) * np.float32(0.1)).astype(np.float32)
    x[1::2] = -x[1::2]
    g = (np.float32(0.25) + (i % 5).astype(np.float32) * np.float32(0.1)).astype(np.float32)
    ss = (x.astype(np.float64) ** 2).sum()
    ref = x.astype(np.float64) / np.sqrt(ss / D + 1e-6) * g.astype(np.float64)
    got = oracle.rms_norm_f32(x[None], g, 1e-6)[0]
    np.testing.assert_allclose(got, ref, rtol=3e-7, atol=0)


def test_sum_of_squares_follows_the_reference_tree(oracle):
    """serenitymojo/ops/norm.mojo:56-72 folds a 256-slot array in halves, far pairs first.  With
    x[0]^2 = 2^24 and 127 ones that order keeps 126 of the 127 ones (only the first partner,
    x[64]^2, is lost to a tie), a left-to-right sum keeps none, and runs of 8 combined
    neighbours-first keep 120 — so the result tells the orders apart."""
    x = np.ones((1, 128), np.float32)
    x[0, 0] = 4096.0
    ss = np.float32(2.0 ** 24 + 126.0)
    inv = np.float32(1.0) / np.sqrt(np.float32(ss / np.float32(128.0)) + np.float32(0.0))
    got = oracle.rms_norm_f32(x, np.ones(128, np.float32), 0.0)
    assert got[0, 1] == np.float32(inv) and got[0, 0] == np.float32(np.float32(4096.0) * inv)
    for wrong in (2.0 ** 24, 2.0 ** 24 + 120.0):
        bad = np.float32(1.0) / np.sqrt(np.float32(np.float32(wrong) / np.float32(128.0)))
        assert got[0, 1] != bad
    # D = 64: slots 64..255 are zero, the first real fold is x[t]^2 + x[t+32]^2
    x64 = np.ones((1, 64), np.float32)
    x64[0, 0] = 4096.0
    ss64 = np.float32(2.0 ** 24 + 62.0)
    inv64 = np.float32(1.0) / np.sqrt(np.float32(ss64 / np.float32(64.0)))
    assert oracle.rms_norm_f32(x64, np.ones(64, np.float32), 0.0)[0, 1] == inv64


def test_properties(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((7, 128)).astype(np.float32)
    ones = np.ones(128, np.float32)
    y = oracle.rms_norm_f32(x, ones, 0.0)
    np.testing.assert_allclose((y.astype(np.float64) ** 2).mean(-1), 1.0, rtol=1e-6)     # unit RMS
    np.testing.assert_array_equal(oracle.rms_norm_f32(2.0 * x, ones, 0.0), y)             # scale-free (power of two: exact)
    # a rotation keeps the length of every pair; angle 0 is the identity; angle pi/2 swaps with a sign
    th = rng.uniform(-3, 3, (7, 64)).astype(np.float32)
    r = oracle.rope_interleaved_f32(x, np.cos(th), np.sin(th))
    np.testing.assert_allclose(r[:, 0::2] ** 2 + r[:, 1::2] ** 2, x[:, 0::2] ** 2 + x[:, 1::2] ** 2, rtol=2e-6)
    np.testing.assert_array_equal(oracle.rope_interleaved_f32(x, np.ones((7, 64)), np.zeros((7, 64))), x)
    q = oracle.rope_interleaved_f32(x, np.zeros((7, 64)), np.ones((7, 64)))
    np.testing.assert_array_equal(q[:, 0::2], -x[:, 1::2])
    np.testing.assert_array_equal(q[:, 1::2], x[:, 0::2])
    # relative-position property: <rope(q, m), rope(k, n)> depends on m - n only
    qv, kv = x[0:1], x[1:2]
    base = 1.0 / (10000.0 ** (np.arange(64) / 64.0))
    def rot(v, pos):
        a = (pos * base)[None].astype(np.float32)
        return oracle.rope_interleaved_f32(v, np.cos(a), np.sin(a)).astype(np.float64)
    d1 = (rot(qv, 5) * rot(kv, 2)).sum()
    d2 = (rot(qv, 13) * rot(kv, 10)).sum()
    assert abs(d1 - d2) < 1e-4 * max(1.0, abs(d1))


@pytest.mark.parametrize("halfsplit", [False, True])
@pytest.mark.parametrize("D,with_rope,batch_rows", [(128, True, 0), (64, True, 0), (128, False, 0), (128, True, 3 * 37)])
def test_bf16_pipeline_matches_numpy_restatement(oracle, D, with_rope, batch_rows, halfsplit):
    rng = np.random.default_rng(11 + D)
    B, S, H = 2, 37, 3
    x = f32_to_bf16_bits(rng.standard_normal((B, S, H, D)).astype(np.float32) * 3.0)
    x[0, 3, 1] = 0                                               # an all-zero row: inv = 1/sqrt(eps), output 0
    gain = f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(D)).astype(np.float32))
    rows = S * H * (B if batch_rows else 1)
    th = rng.uniform(-3.14, 3.14, (rows, D // 2))
    cos, sin = (np.cos(th).astype(np.float32), np.sin(th).astype(np.float32)) if with_rope else (None, None)
    got = oracle.norm_rope_bf16(x, gain, 1e-6, cos, sin, batch_rows, halfsplit=halfsplit)
    want = R.norm_rope_bf16(x, gain, 1e-6, cos, sin, batch_rows, halfsplit=halfsplit)
    np.testing.assert_array_equal(got, want)
    assert not bf16_bits_to_f32(got[0, 3, 1]).any()                 # (signed zeros allowed)
    # and it is the composition of the two fp32 ops with a bf16 store in between, to bf16 precision
    xf = bf16_bits_to_f32(x).reshape(-1, D)
    y = oracle.rms_norm_f32(xf, bf16_bits_to_f32(gain), 1e-6)
    if with_rope:
        idx = (np.arange(B)[:, None, None] * batch_rows + np.arange(S)[None, :, None] * H + np.arange(H)[None, None, :]).reshape(-1)
        y = (oracle.rope_halfsplit_f32 if halfsplit else oracle.rope_interleaved_f32)(y, cos[idx], sin[idx])
    # (a rotated pair can cancel, so the bf16 steps of the inputs show as absolute error)
    np.testing.assert_allclose(bf16_bits_to_f32(got).reshape(-1, D), y, rtol=2.0 ** -6, atol=3e-2)


@pytest.mark.parametrize("H,D", [(32, 128), (5, 64)])
def test_full_row_norm_halfsplit_bf16_tables(oracle, H, D):
    """The pre-attention sequence of serenitymojo/models/ltx2/ltx2_block.mojo:419-432: rms_norm over
    the whole inner dim H*D (gain [H*D]), reshape to heads, rope_halfsplit with bf16 tables.  Against
    the numpy restatement bit for bit, and against the composition of the checker's fp32 ops."""
    rng = np.random.default_rng(5 + H)
    B, S = 2, 9
    x = f32_to_bf16_bits(rng.standard_normal((B, S, H, D)).astype(np.float32) * 2.0)
    x[1, 4] = 0                                                  # an all-zero token
    gain = f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(H * D)).astype(np.float32))
    th = rng.uniform(-3.14, 3.14, (S * H, D // 2))
    cos, sin = f32_to_bf16_bits(np.cos(th).astype(np.float32)), f32_to_bf16_bits(np.sin(th).astype(np.float32))
    got = oracle.norm_rope_bf16(x, gain, 1e-6, cos, sin, 0, halfsplit=True, full_row=True)
    want = R.norm_rope_bf16(x, gain, 1e-6, cos, sin, 0, halfsplit=True, full_row=True)
    np.testing.assert_array_equal(got, want)
    assert not bf16_bits_to_f32(got[1, 4]).any()
    y = oracle.rms_norm_f32(bf16_bits_to_f32(x).reshape(B * S, H * D), bf16_bits_to_f32(gain), 1e-6).reshape(B * S * H, D)
    idx = np.tile(np.arange(S * H), B)
    y = oracle.rope_halfsplit_f32(y, bf16_bits_to_f32(cos)[idx], bf16_bits_to_f32(sin)[idx])
    np.testing.assert_allclose(bf16_bits_to_f32(got).reshape(-1, D), y, rtol=2.0 ** -6, atol=3e-2)
    # the statistic really is the row's: scaling one head changes every head's output
    x2 = x.copy()
    x2[:, :, 0] = f32_to_bf16_bits(bf16_bits_to_f32(x[:, :, 0]) * 4.0)
    got2 = oracle.norm_rope_bf16(x2, gain, 1e-6, cos, sin, 0, halfsplit=True, full_row=True)
    assert (got2[0, 0, 1] != got[0, 0, 1]).any()
