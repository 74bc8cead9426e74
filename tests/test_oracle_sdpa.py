"""Pins the oracle's full-precision SDPA (the referee) against the golden
vectors the reference's own tests hold, closed forms and a library routine."""
import json
import os

import numpy as np
import torch

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _closed_form_qkv(B, S, H, D):
    """serenitymojo/ops/parity/sdpa_math_parity.mojo:32-50 (BSHD flat index i)."""
    i = np.arange(B * S * H * D, dtype=np.int64)
    q = (((i * 7) % 13).astype(np.float64) - 6.0) * 0.05
    k = (((i * 5) % 11).astype(np.float64) - 5.0) * 0.05
    v = (((i * 3) % 9).astype(np.float64) - 4.0) * 0.05
    shp = (B, S, H, D)
    return q.reshape(shp), k.reshape(shp), v.reshape(shp)


def test_golden_sdpa_math_ref_dh128(oracle):
    ref = np.load(os.path.join(GOLD, "sdpa_math_ref.npz"))["dh128"]
    B, S, H, D = 1, 8, 32, 128
    q, k, v = _closed_form_qkv(B, S, H, D)
    o = oracle.sdpa_f32(q, k, v, float(1.0 / np.sqrt(D)))
    # fixture is printed with %.8f; inputs here are fp32-rounded
    np.testing.assert_allclose(o.reshape(-1), ref, atol=2e-7, rtol=0)
    o2 = oracle.sdpa_f32(q, k, v, float(1.0 / np.sqrt(D)), online=True)
    np.testing.assert_allclose(o2.reshape(-1), ref, atol=2e-6, rtol=0)


def test_golden_sdpa_math_ref_dh512(oracle):
    ref = np.load(os.path.join(GOLD, "sdpa_math_ref.npz"))["dh512"]
    B, S, H, D = 1, 64, 1, 512
    q, k, v = _closed_form_qkv(B, S, H, D)
    o = oracle.sdpa_f32(q, k, v, float(1.0 / np.sqrt(D)))
    np.testing.assert_allclose(o.reshape(-1), ref, atol=2e-7, rtol=0)


def test_golden_ops_smoke2_kat(oracle):
    """serenitymojo/ops_smoke2.mojo:239-302: randn inputs, H>1 BSHD indexing."""
    with open(os.path.join(GOLD, "ops_smoke2_sdpa_kat.json")) as f:
        kat = json.load(f)
    shp = kat["shape_bshd"]
    q, k, v = (np.float32(kat[n]).reshape(shp) for n in ("q_sdpa", "k_sdpa", "v_sdpa"))
    want = np.float32(kat["out_sdpa_ref"]).reshape(shp)
    for online in (False, True):
        o = oracle.sdpa_f32(q, k, v, kat["scale"], online=online)
        np.testing.assert_allclose(o, want, atol=5e-7, rtol=0)


def test_closed_forms(oracle):
    rng = np.random.default_rng(7)
    B, S, H, D = 2, 37, 3, 16
    q = rng.standard_normal((B, S, H, D)).astype(np.float32)
    v = rng.standard_normal((B, S, H, D)).astype(np.float32)
    # identical K rows -> uniform softmax -> out = mean(V) over tokens
    k = np.broadcast_to(rng.standard_normal((B, 1, H, D)).astype(np.float32), (B, S, H, D))
    o = oracle.sdpa_f32(q, k, v, 0.3)
    np.testing.assert_allclose(o, np.broadcast_to(v.astype(np.float64).mean(1, keepdims=True), o.shape), atol=1e-6)
    # constant V -> out = V
    k = rng.standard_normal((B, S, H, D)).astype(np.float32)
    vc = np.broadcast_to(rng.standard_normal((B, 1, H, D)).astype(np.float32), (B, S, H, D))
    np.testing.assert_allclose(oracle.sdpa_f32(q, k, vc, 0.3), vc, atol=1e-6)
    # one-hot q.k with a large scale -> out -> V[argmax]
    D2 = S
    eye = np.zeros((B, S, H, D2), np.float32)
    for s in range(S):
        eye[:, s, :, s] = 1.0
    v2 = rng.standard_normal((B, S, H, D2)).astype(np.float32)
    perm = rng.permutation(S)
    o = oracle.sdpa_f32(eye[:, perm], eye, v2, 200.0)
    np.testing.assert_allclose(o, v2[:, perm], atol=1e-6)
    # adding a constant vector to every K row leaves the output unchanged (K smoothing identity)
    mu = rng.standard_normal((B, 1, H, D)).astype(np.float32)
    o_a = oracle.sdpa_f32(q, k, v, 0.3)
    o_b = oracle.sdpa_f32(q, k + mu, v, 0.3)
    np.testing.assert_allclose(o_a, o_b, atol=2e-5)


def test_against_library_and_rectangular(oracle):
    rng = np.random.default_rng(8)
    B, Sq, Skv, H, D = 2, 50, 131, 4, 64
    q = rng.standard_normal((B, Sq, H, D)).astype(np.float32)
    k = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
    v = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
    scale = 0.11
    want = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q).permute(0, 2, 1, 3).double(), torch.from_numpy(k).permute(0, 2, 1, 3).double(),
        torch.from_numpy(v).permute(0, 2, 1, 3).double(), scale=scale).permute(0, 2, 1, 3).numpy()
    np.testing.assert_allclose(oracle.sdpa_f32(q, k, v, scale), want, atol=1e-6)
    np.testing.assert_allclose(oracle.sdpa_f32(q, k, v, scale, online=True), want, atol=1e-5)


def test_brute_force_float64_tiny(oracle):
    rng = np.random.default_rng(9)
    B, S, H, D = 1, 5, 2, 3
    q, k, v = (rng.standard_normal((B, S, H, D)).astype(np.float32) for _ in range(3))
    want = np.zeros((B, S, H, D))
    for h in range(H):
        for i in range(S):
            s = np.array([0.7 * sum(float(q[0, i, h, d]) * float(k[0, j, h, d]) for d in range(D)) for j in range(S)])
            p = np.exp(s - s.max())
            p /= p.sum()
            for d in range(D):
                want[0, i, h, d] = sum(p[j] * float(v[0, j, h, d]) for j in range(S))
    np.testing.assert_allclose(oracle.sdpa_f32(q, k, v, 0.7), want, atol=1e-6)


def test_bad_args(oracle):
    import ctypes
    L = oracle.lib()
    st = oracle.strides_bshd(4, 1, 8)
    x = np.zeros(32, np.float32)
    p = x.ctypes.data_as(ctypes.c_void_p)
    assert L.sage_oracle_sdpa_f32(None, p, p, p, 1, 1, 4, 4, 8, 1.0, st, st, st, st) == -1
    assert L.sage_oracle_sdpa_f32(p, p, p, p, 1, 0, 4, 4, 8, 1.0, st, st, st, st) == -1
    assert L.sage_oracle_sdpa_f32(p, p, p, p, 1, 1, 4, 4, 8, 1.0, None, st, st, st) == -1
