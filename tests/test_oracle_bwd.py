"""Pins the oracle's SDPA backward against the gradients the reference's own parity test holds,
torch.autograd in float64, central differences and invariants of softmax attention."""
import os

import numpy as np
import torch

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _closed_form_qkv_dout(B, S, H, D):
    """serenitymojo/ops/parity/sdpa_bwd_parity.mojo:44-65 (BSHD flat index i)."""
    i = np.arange(B * S * H * D, dtype=np.int64)
    q = (((i * 7) % 13).astype(np.float64) - 6.0) * 0.05
    k = (((i * 5) % 11).astype(np.float64) - 5.0) * 0.05
    v = (((i * 3) % 9).astype(np.float64) - 4.0) * 0.05
    g = (((i * 2) % 7).astype(np.float64) - 3.0) * 0.05
    shp = (B, S, H, D)
    return q.reshape(shp), k.reshape(shp), v.reshape(shp), g.reshape(shp)


def _torch_grads(q, k, v, g, scale, nq=None, nk=None):
    """float64 autograd of softmax(q k^T scale) v on the valid part; padding rows get zero."""
    Q, K, V = (torch.tensor(np.asarray(t, np.float64), requires_grad=True) for t in (q, k, v))
    G = torch.tensor(np.asarray(g, np.float64))
    nq = Q.shape[1] if nq is None else nq
    nk = K.shape[1] if nk is None else nk
    s = scale * torch.einsum("bihd,bjhd->bhij", Q[:, :nq], K[:, :nk])
    out = torch.einsum("bhij,bjhd->bihd", torch.softmax(s, dim=-1), V[:, :nk])
    out.backward(G[:, :nq])
    return Q.grad.numpy(), K.grad.numpy(), V.grad.numpy()


def test_golden_sdpa_bwd_ref(oracle):
    """ops/parity/sdpa_bwd_ref.txt: dh128 [1,8,32,128] and dh64 [1,8,8,64], printed with %.8f."""
    ref = np.load(os.path.join(GOLD, "sdpa_bwd_ref.npz"))
    for tag, (B, S, H, D) in (("dh128", (1, 8, 32, 128)), ("dh64", (1, 8, 8, 64))):
        q, k, v, g = _closed_form_qkv_dout(B, S, H, D)
        dq, dk, dv = oracle.sdpa_bwd_f32(q, k, v, g, float(1.0 / np.sqrt(D)))
        for name, got in (("dq", dq), ("dk", dk), ("dv", dv)):
            want = ref[tag + "_" + name]
            assert np.abs(want).max() > 1e-5          # not a comparison of zeros
            np.testing.assert_allclose(got.reshape(-1), want, atol=6e-9, rtol=2e-6, err_msg=tag + "_" + name)


def test_against_torch_autograd_float64(oracle):
    rng = np.random.default_rng(11)
    for (B, Sq, Skv, H, D, scale) in ((2, 37, 37, 3, 16, 0.25), (1, 64, 77, 5, 64, 0.125), (1, 96, 16, 4, 128, 0.0884)):
        q = rng.standard_normal((B, Sq, H, D)).astype(np.float32)
        k = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
        v = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
        g = rng.standard_normal((B, Sq, H, D)).astype(np.float32)
        want = _torch_grads(q, k, v, g, scale)
        got = oracle.sdpa_bwd_f32(q, k, v, g, scale)
        for a, b in zip(got, want):
            np.testing.assert_allclose(a, b, atol=2e-6, rtol=2e-6)


def test_flash_form_equals_recompute_form(oracle):
    """With the exact output and log-sum-exp handed in, exp(score - lse) and rowsum(dO * O) are the
    softmax and its backward row term: the two forms agree to fp32 rounding of o and stats."""
    rng = np.random.default_rng(12)
    B, Sq, Skv, H, D, scale = 1, 50, 70, 2, 32, 0.2
    q = rng.standard_normal((B, Sq, H, D)).astype(np.float32)
    k = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
    v = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
    g = rng.standard_normal((B, Sq, H, D)).astype(np.float32)
    o, stats = oracle.sdpa_f32(q, k, v, scale, want_stats=True)
    a = oracle.sdpa_bwd_f32(q, k, v, g, scale)
    b = oracle.sdpa_bwd_f32(q, k, v, g, scale, o=o, stats=stats)
    for x, y in zip(a, b):
        np.testing.assert_allclose(x, y, atol=3e-6, rtol=1e-5)
    # a wrong log-sum-exp is NOT silently renormalised: the probabilities scale by exp(-shift)
    c = oracle.sdpa_bwd_f32(q, k, v, g, scale, o=o, stats=stats + np.float32(np.log(2.0)))
    np.testing.assert_allclose(c[2], 0.5 * a[2], atol=3e-6, rtol=1e-5)


def test_central_differences(oracle):
    """d/dx of L = sum(dout * sdpa(q,k,v)) by central differences on a few coordinates (float64
    forward written here, independent of the oracle's code)."""
    rng = np.random.default_rng(13)
    B, Sq, Skv, H, D, scale = 1, 5, 7, 2, 4, 0.6
    q = rng.standard_normal((B, Sq, H, D))
    k = rng.standard_normal((B, Skv, H, D))
    v = rng.standard_normal((B, Skv, H, D))
    g = rng.standard_normal((B, Sq, H, D))

    def loss(q, k, v):
        s = scale * np.einsum("bihd,bjhd->bhij", q, k)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        return float((np.einsum("bhij,bjhd->bihd", p, v) * g).sum())

    dq, dk, dv = oracle.sdpa_bwd_f32(q, k, v, g, scale)
    eps = 1e-4
    for arr, grad, which in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
        for idx in [(0, 0, 0, 0), (0, arr.shape[1] - 1, 1, 3), (0, 2, 1, 1)]:
            hi, lo = [q.copy(), k.copy(), v.copy()], [q.copy(), k.copy(), v.copy()]
            hi[which][idx] += eps
            lo[which][idx] -= eps
            fd = (loss(*hi) - loss(*lo)) / (2 * eps)
            # inputs reach the oracle as fp32
            assert abs(fd - grad[idx]) < 2e-5 * max(1.0, abs(fd)), (which, idx, fd, grad[idx])


def test_invariants(oracle):
    rng = np.random.default_rng(14)
    B, Sq, Skv, H, D, scale = 2, 33, 41, 3, 16, 0.3
    q = rng.standard_normal((B, Sq, H, D)).astype(np.float32)
    k = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
    v = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
    g = rng.standard_normal((B, Sq, H, D)).astype(np.float32)
    dq, dk, dv = oracle.sdpa_bwd_f32(q, k, v, g, scale)
    # attention does not change when every key moves by the same vector: sum_j dK_j = 0
    assert np.abs(dk.sum(axis=1)).max() < 1e-5
    # probabilities of a row sum to one: sum_j dV_j = sum_i dO_i
    np.testing.assert_allclose(dv.sum(axis=1), g.sum(axis=1), atol=2e-5)
    # the output is linear in v and in dout
    dq2, dk2, dv2 = oracle.sdpa_bwd_f32(q, k, 2 * v, 3 * g, scale)
    np.testing.assert_allclose(dq2, 6 * dq, atol=1e-5, rtol=1e-5)
    np.testing.assert_allclose(dk2, 6 * dk, atol=1e-5, rtol=1e-5)
    np.testing.assert_allclose(dv2, 3 * dv, atol=1e-5, rtol=1e-5)
    # identical keys: uniform attention, no gradient reaches q; dV_j = mean-weight * sum_i dO_i
    k1 = np.broadcast_to(k[:, :1], k.shape).copy()
    dq3, dk3, dv3 = oracle.sdpa_bwd_f32(q, k1, v, g, scale)
    assert np.abs(dq3).max() < 1e-6
    np.testing.assert_allclose(dv3, np.broadcast_to(g.sum(axis=1, keepdims=True) / Skv, v.shape), atol=1e-5)


def test_valid_lengths(oracle):
    """real_N_q / real_N_kv of cudnn_sdpa_bwd.cpp:344: padding rows and keys take no part."""
    rng = np.random.default_rng(15)
    B, Sq, Skv, H, D, scale = 1, 48, 64, 2, 32, 0.2
    nq, nk = 37, 51
    q = rng.standard_normal((B, Sq, H, D)).astype(np.float32)
    k = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
    v = rng.standard_normal((B, Skv, H, D)).astype(np.float32)
    g = rng.standard_normal((B, Sq, H, D)).astype(np.float32)
    want = _torch_grads(q, k, v, g, scale, nq, nk)
    got = oracle.sdpa_bwd_f32(q, k, v, g, scale, real_nq=nq, real_nkv=nk)
    for a, b in zip(got, want):
        np.testing.assert_allclose(a, b, atol=2e-6, rtol=2e-6)
    assert not got[0][:, nq:].any() and not got[1][:, nk:].any() and not got[2][:, nk:].any()
    # flash form with the masked forward's output and log-sum-exp
    o, stats = oracle.sdpa_f32(q, k, v, scale, mask_lo=nk, mask_hi=Skv, want_stats=True)
    got2 = oracle.sdpa_bwd_f32(q, k, v, g, scale, o=o, stats=stats, real_nq=nq, real_nkv=nk)
    for a, b in zip(got2, want):
        np.testing.assert_allclose(a, b, atol=3e-6, rtol=1e-5)


def test_flash_form_after_the_quantized_forward(oracle):
    """O and stats from the quantized forward are consistent with ITS probabilities, not with the
    exact ones the backward recomputes: the rows of dS then sum to a small non-zero number.  With keys
    that share a large offset (workload 2) the uncentred dS K would multiply that number by the offset
    (cosine of dQ against the exact gradient 0.9987); centred keys keep every gradient at 0.9999."""
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    from mojodiffusion_amd.workloads import WORKLOADS, make_inputs, bf16_bits_to_f32
    w = WORKLOADS[2].scaled(B=1, H=2, S=320)
    q, k, v = make_inputs(w)
    qf, kf, vf = (bf16_bits_to_f32(t) for t in (q, k, v))
    g = np.random.default_rng(3).standard_normal(q.shape).astype(np.float32)
    ob, _, stats = oracle.sdpa_bf16(q, k, v, w.scale, variant=0, blkq=128, blkk=64, want_stats=True)
    exact = oracle.sdpa_bwd_f32(qf, kf, vf, g, w.scale)
    got = oracle.sdpa_bwd_f32(qf, kf, vf, g, w.scale, o=bf16_bits_to_f32(ob), stats=stats)
    for a, b in zip(got, exact):
        a, b = a.astype(np.float64).reshape(-1), b.astype(np.float64).reshape(-1)
        assert a @ b / np.sqrt((a @ a) * (b @ b)) >= 0.9999
    # the uncentred product, written out here, is what loses it
    s = w.scale * np.einsum("bihd,bjhd->bhij", qf.astype(np.float64), kf.astype(np.float64))
    P = np.exp(s - stats[..., None].astype(np.float64))
    dP = np.einsum("bihd,bjhd->bhij", g.astype(np.float64), vf.astype(np.float64))
    delta = np.einsum("bihd,bihd->bhi", g.astype(np.float64), bf16_bits_to_f32(ob).astype(np.float64))
    dq = w.scale * np.einsum("bhij,bjhd->bihd", P * (dP - delta[..., None]), kf.astype(np.float64)).reshape(-1)
    e = exact[0].astype(np.float64).reshape(-1)
    assert dq @ e / np.sqrt((dq @ dq) * (e @ e)) < 0.9995
