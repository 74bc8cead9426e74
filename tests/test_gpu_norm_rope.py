"""GPU parity of the quantizers with RMSNorm + interleaved RoPE fused in front: the INT8 codes,
scales and the K statistics must be bit-identical with what the CPU checker gets by running its
norm/rope restatement first and its quantizers on the result; the one-shot call must agree with
the unfused pipeline."""
import numpy as np
import pytest

from mojodiffusion_amd import _lib
from mojodiffusion_amd.workloads import WORKLOADS, make_inputs, f32_to_bf16_bits, bf16_bits_to_f32

pytestmark = pytest.mark.gpu


def _tables(rng, rows, D):
    """RoPE tables of the sampler's shape: one angle per (row, pair)."""
    th = rng.uniform(-np.pi, np.pi, (rows, D // 2))
    return np.cos(th).astype(np.float32), np.sin(th).astype(np.float32)


def _gains(rng, D):
    return (f32_to_bf16_bits((1.0 + 0.3 * rng.standard_normal(D)).astype(np.float32)),
            f32_to_bf16_bits((0.7 + 0.3 * rng.standard_normal(D)).astype(np.float32)))


def _gpu_quant(q, k, scale, blkq, blkk, smooth, gq, gk, eps, cos, sin, batch_rows, halfsplit=False, full_row=False):
    import torch
    import gpu_harness as H
    L = _lib.lib()
    B, S, Hh, D = q.shape
    qd, kd = H.dev_bf16(q), H.dev_bf16(k)
    gqd, gkd = H.dev_bf16(gq), H.dev_bf16(gk)
    tab16 = cos is not None and cos.dtype == np.uint16
    cd = (H.dev_bf16(cos) if tab16 else torch.from_numpy(cos).cuda()) if cos is not None else None
    sd = (H.dev_bf16(sin) if tab16 else torch.from_numpy(sin).cuda()) if sin is not None else None
    nqp, nkp = L.mi355_sage_pad_q(S), L.mi355_sage_pad_kv(S)
    q8 = torch.full((B, Hh, nqp, D), 77, dtype=torch.int8, device="cuda")
    k8 = torch.full((B, Hh, nkp, D), 77, dtype=torch.int8, device="cuda")
    qs = torch.full((B, Hh, nqp // blkq), -1.0, dtype=torch.float32, device="cuda")
    ks = torch.full((B, Hh, nkp // blkk), -1.0, dtype=torch.float32, device="cuda")
    km, qm, kmu = (torch.full((B, Hh, D), -1.0, dtype=torch.float32, device="cuda") for _ in range(3))
    scr = torch.empty(max(L.mi355_sage_quant_scratch_bytes(B, Hh, S, D), 8), dtype=torch.uint8, device="cuda")
    st = _lib.strides_bhnd(S, Hh, D)
    rc = L.mi355_sage_quant_qk_norm_rope_bf16(
        qd.data_ptr(), kd.data_ptr(), B, Hh, S, S, D, scale, st, st, 0, 0,
        gqd.data_ptr(), gkd.data_ptr(), eps, cd.data_ptr() if cd is not None else None,
        sd.data_ptr() if sd is not None else None, batch_rows,
        (1 if halfsplit else 0) | (2 if tab16 else 0) | (4 if full_row else 0), blkq, blkk, (1 if smooth else 0) | 2,
        q8.data_ptr(), qs.data_ptr(), k8.data_ptr(), ks.data_ptr(), km.data_ptr(), qm.data_ptr(), kmu.data_ptr(),
        scr.data_ptr(), scr.numel(), H.stream())
    assert rc == 0, rc
    torch.cuda.synchronize()
    return dict(q8=q8.cpu().numpy(), qscale=qs.cpu().numpy(), k8=k8.cpu().numpy(), kscale=ks.cpu().numpy(),
                kmean=km.cpu().numpy(), qmul=qm.cpu().numpy(), kmul=kmu.cpu().numpy())


@pytest.mark.parametrize("halfsplit", [False, True])
@pytest.mark.parametrize("D,S,blkq,blkk,smooth,rope,per_batch", [
    (128, 300, 128, 64, True, True, False), (128, 1100, 128, 64, True, True, True),
    (64, 200, 64, 64, True, True, False), (128, 77, 32, 32, False, True, False),
    (128, 513, 128, 64, True, False, False), (64, 1, 32, 32, True, True, False)])
def test_fused_quantizers_bit_exact(oracle, D, S, blkq, blkk, smooth, rope, per_batch, halfsplit):
    if halfsplit and not rope:
        pytest.skip("the pairing only matters with tables")
    rng = np.random.default_rng(100 + S)
    B, Hh = 2, 3
    q = f32_to_bf16_bits(rng.standard_normal((B, S, Hh, D)).astype(np.float32) * 2.0)
    k = f32_to_bf16_bits((rng.standard_normal((B, S, Hh, D)) + 1.5 * rng.standard_normal((B, 1, Hh, D))).astype(np.float32))
    if S > 5:
        q[1, 3, 0] = 0                                         # an all-zero row
    gq, gk = _gains(rng, D)
    cos, sin = _tables(rng, S * Hh * (B if per_batch else 1), D) if rope else (None, None)
    batch_rows = S * Hh if per_batch else 0
    eps, scale = 1e-6, 1.0 / np.sqrt(D)
    got = _gpu_quant(q, k, scale, blkq, blkk, smooth, gq, gk, eps, cos, sin, batch_rows, halfsplit)
    qn = oracle.norm_rope_bf16(q, gq, eps, cos, sin, batch_rows, halfsplit=halfsplit)
    kn = oracle.norm_rope_bf16(k, gk, eps, cos, sin, batch_rows, halfsplit=halfsplit)
    import gpu_harness as H
    want = H.oracle_quant_qk(oracle, qn, kn, scale, blkq, blkk, smooth, True)
    for name in ("kmean", "qmul", "kmul"):
        np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    nqb, nkb = want["qscale"].shape[2], want["kscale"].shape[2]
    np.testing.assert_array_equal(got["qscale"][:, :, :nqb].view(np.uint32), want["qscale"].view(np.uint32))
    np.testing.assert_array_equal(got["kscale"][:, :, :nkb].view(np.uint32), want["kscale"].view(np.uint32))
    np.testing.assert_array_equal(got["q8"], want["q8"])
    np.testing.assert_array_equal(got["k8"], want["k8"])


@pytest.mark.parametrize("variant,wid,halfsplit", [(0, 2, False), (1, 2, False), (0, 1, False), (0, 2, True), (1, 1, True)])
def test_one_shot_equals_unfused_pipeline(oracle, variant, wid, halfsplit):
    """mi355_sage_sdpa_bf16_norm_rope on the projections == the plain one-shot call on
    norm/rope'd tensors (the CPU checker's, which the test above proves equal to the fused
    kernels' view bit for bit): same quantized tensors, hence the same output bits."""
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    rng = np.random.default_rng(9)
    w = WORKLOADS[wid].scaled(B=2 if wid == 1 else 1, H=3, S=700)      # wid 1: head dim 64
    q, k, v = make_inputs(w)
    gq, gk = _gains(rng, w.D)
    cos, sin = _tables(rng, w.S * w.H, w.D)
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    got = A.qk_norm_rope_sdpa_nomask(qd, kd, vd, H.dev_bf16(gq), H.dev_bf16(gk), 1e-6,
                                     torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda(), w.scale, variant,
                                     blkq=w.blkq, blkk=w.blkk, halfsplit=halfsplit)
    torch.cuda.synchronize()
    qn = oracle.norm_rope_bf16(q, gq, 1e-6, cos, sin, 0, halfsplit=halfsplit)
    kn = oracle.norm_rope_bf16(k, gk, 1e-6, cos, sin, 0, halfsplit=halfsplit)
    want = torch.empty_like(qd)
    st = _lib.strides_bhnd(w.S, w.H, w.D)
    qnd, knd = H.dev_bf16(qn), H.dev_bf16(kn)
    rc = _lib.lib().mi355_sage_sdpa_bf16_ex(qnd.data_ptr(), knd.data_ptr(), vd.data_ptr(), want.data_ptr(),
                                            w.B, w.H, w.S, w.S, w.D, w.scale, st, st, st, st, 0, 0, 0, 0, 0, H.stream(),
                                            variant, w.blkq, w.blkk, 3, None, 0)
    assert rc == 0, rc
    torch.cuda.synchronize()
    np.testing.assert_array_equal(H.to_bits(got), H.to_bits(want))
    # and against an fp32 attention on the fp32 norm/rope
    cb, sb = np.tile(cos, (w.B, 1)), np.tile(sin, (w.B, 1))      # the table is shared by the batches
    rope = oracle.rope_halfsplit_f32 if halfsplit else oracle.rope_interleaved_f32
    qf = rope(oracle.rms_norm_f32(bf16_bits_to_f32(q).reshape(-1, w.D), bf16_bits_to_f32(gq), 1e-6), cb, sb)
    kf = rope(oracle.rms_norm_f32(bf16_bits_to_f32(k).reshape(-1, w.D), bf16_bits_to_f32(gk), 1e-6), cb, sb)
    ref = oracle.sdpa_f32(qf.reshape(q.shape), kf.reshape(k.shape), bf16_bits_to_f32(v), w.scale)
    cos_sim, mx = H.cos_maxabs(got.float().cpu().numpy(), ref)
    assert cos_sim >= 0.999, (cos_sim, mx)


def test_argument_errors():
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    x = torch.zeros((1, 64, 2, 128), dtype=torch.bfloat16, device="cuda")
    g = torch.ones(128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(A.Error):
        A.qk_norm_rope_sdpa_nomask(x, x, x, g[:64], g, 1e-6, None, None, 0.1)
    with pytest.raises(A.Error):
        A.qk_norm_rope_sdpa_nomask(x, x, x, g, g, 1e-6, torch.zeros((5, 64), device="cuda"), torch.zeros((5, 64), device="cuda"), 0.1)
    L = _lib.lib()
    st = _lib.strides_bhnd(64, 2, 128)
    o = torch.empty_like(x)
    # gains missing -> -1; misaligned gain -> -2
    rc = L.mi355_sage_sdpa_bf16_norm_rope(x.data_ptr(), x.data_ptr(), x.data_ptr(), o.data_ptr(), 1, 2, 64, 64, 128, 0.1,
                                          st, st, st, st, 0, 0, 0, 0, 0, H.stream(), 0, 128, 64, 1,
                                          None, None, 1e-6, None, None, 0, 0, None, 0)
    assert rc == -1
    rc = L.mi355_sage_sdpa_bf16_norm_rope(x.data_ptr(), x.data_ptr(), x.data_ptr(), o.data_ptr(), 1, 2, 64, 64, 128, 0.1,
                                          st, st, st, st, 0, 0, 0, 0, 0, H.stream(), 0, 128, 64, 1,
                                          g.data_ptr() + 2, g.data_ptr(), 1e-6, None, None, 0, 0, None, 0)
    assert rc == -2
    # the table has one row per position, shared by Q and K: N_q != N_kv is refused (-2), norm only is fine
    t = torch.zeros((64 * 2, 64), dtype=torch.float32, device="cuda")
    st32 = _lib.strides_bhnd(32, 2, 128)
    rc = L.mi355_sage_sdpa_bf16_norm_rope(x.data_ptr(), x.data_ptr(), x.data_ptr(), o.data_ptr(), 1, 2, 32, 64, 128, 0.1,
                                          st32, st, st, st32, 0, 0, 0, 0, 0, H.stream(), 0, 128, 64, 3,
                                          g.data_ptr(), g.data_ptr(), 1e-6, t.data_ptr(), t.data_ptr(), 0, 0, None, 0)
    assert rc == -2
    rc = L.mi355_sage_sdpa_bf16_norm_rope(x.data_ptr(), x.data_ptr(), x.data_ptr(), o.data_ptr(), 1, 2, 32, 64, 128, 0.1,
                                          st32, st, st, st32, 0, 0, 0, 0, 0, H.stream(), 0, 128, 64, 3,
                                          g.data_ptr(), g.data_ptr(), 1e-6, None, None, 0, 0, None, 0)
    assert rc == 0
    # an unknown option bit is refused
    rc = L.mi355_sage_sdpa_bf16_norm_rope(x.data_ptr(), x.data_ptr(), x.data_ptr(), o.data_ptr(), 1, 2, 64, 64, 128, 0.1,
                                          st, st, st, st, 0, 0, 0, 0, 0, H.stream(), 0, 128, 64, 3,
                                          g.data_ptr(), g.data_ptr(), 1e-6, None, None, 0, 8, None, 0)
    assert rc == -1
    torch.cuda.synchronize()


def test_fused_train_fwd_stats(oracle):
    """Stats of the fused call = natural-log LSE of the scaled scores of the normalised, rotated
    Q and K (computed here in float64 from the checker's bf16 norm/rope output), and O equals the
    fused inference call bit for bit."""
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    rng = np.random.default_rng(21)
    w = WORKLOADS[2].scaled(B=1, H=2, S=384)
    q, k, v = make_inputs(w)
    gq, gk = _gains(rng, w.D)
    cos, sin = _tables(rng, w.S * w.H, w.D)
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    gqd, gkd = H.dev_bf16(gq), H.dev_bf16(gk)
    cd, sd = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    fwd = A.qk_norm_rope_sdpa_flash_train_fwd(qd, kd, vd, gqd, gkd, 1e-6, cd, sd, w.scale)
    inf = A.qk_norm_rope_sdpa_nomask(qd, kd, vd, gqd, gkd, 1e-6, cd, sd, w.scale)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(H.to_bits(fwd.o), H.to_bits(inf))
    qn = bf16_bits_to_f32(oracle.norm_rope_bf16(q, gq, 1e-6, cos, sin, 0)).astype(np.float64)
    kn = bf16_bits_to_f32(oracle.norm_rope_bf16(k, gk, 1e-6, cos, sin, 0)).astype(np.float64)
    s = np.einsum("bihd,bjhd->bhij", qn, kn) * w.scale
    lse = np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1)) + s.max(-1)
    np.testing.assert_allclose(fwd.stats.cpu().numpy()[..., 0], lse, atol=3e-2)


@pytest.mark.parametrize("Hh,D,S", [(32, 128, 70), (5, 64, 130)])
def test_full_row_norm_halfsplit_bf16_tables_bit_exact(oracle, Hh, D, S):
    """LTX-2's pre-attention sequence (models/ltx2/ltx2_block.mojo:419-432) fused into the quantizers:
    RMSNorm over the whole inner dim H*D with a gain of H*D entries, half-split RoPE with bf16
    tables.  INT8 codes, scales and K statistics against the checker run on the checker's own
    norm/rope output, bit for bit; and the one-shot call against the plain call on that output."""
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    rng = np.random.default_rng(40 + Hh)
    B = 2
    q = f32_to_bf16_bits(rng.standard_normal((B, S, Hh, D)).astype(np.float32) * 2.0)
    k = f32_to_bf16_bits((rng.standard_normal((B, S, Hh, D)) + 1.5 * rng.standard_normal((B, 1, Hh, D))).astype(np.float32))
    v = f32_to_bf16_bits(rng.standard_normal((B, S, Hh, D)).astype(np.float32))
    q[1, 3] = 0                                                # an all-zero token
    gq = f32_to_bf16_bits((1.0 + 0.3 * rng.standard_normal(Hh * D)).astype(np.float32))
    gk = f32_to_bf16_bits((0.7 + 0.3 * rng.standard_normal(Hh * D)).astype(np.float32))
    th = rng.uniform(-3.14, 3.14, (S * Hh, D // 2))
    cos, sin = f32_to_bf16_bits(np.cos(th).astype(np.float32)), f32_to_bf16_bits(np.sin(th).astype(np.float32))
    eps, scale = 1e-6, 1.0 / np.sqrt(D)
    got = _gpu_quant(q, k, scale, 128, 64, True, gq, gk, eps, cos, sin, 0, halfsplit=True, full_row=True)
    qn = oracle.norm_rope_bf16(q, gq, eps, cos, sin, 0, halfsplit=True, full_row=True)
    kn = oracle.norm_rope_bf16(k, gk, eps, cos, sin, 0, halfsplit=True, full_row=True)
    want = H.oracle_quant_qk(oracle, qn, kn, scale, 128, 64, True, True)
    for name in ("kmean", "qmul", "kmul"):
        np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    nqb, nkb = want["qscale"].shape[2], want["kscale"].shape[2]
    np.testing.assert_array_equal(got["qscale"][:, :, :nqb].view(np.uint32), want["qscale"].view(np.uint32))
    np.testing.assert_array_equal(got["kscale"][:, :, :nkb].view(np.uint32), want["kscale"].view(np.uint32))
    np.testing.assert_array_equal(got["q8"], want["q8"])
    np.testing.assert_array_equal(got["k8"], want["k8"])
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    fused = A.qk_norm_rope_sdpa_nomask(qd, kd, vd, H.dev_bf16(gq), H.dev_bf16(gk), eps, H.dev_bf16(cos), H.dev_bf16(sin),
                                       scale, halfsplit=True, full_row=True)
    plain = A.sdpa_nomask(H.dev_bf16(qn), H.dev_bf16(kn), vd, scale)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(H.to_bits(fused), H.to_bits(plain))
    with pytest.raises(A.Error, match="weight must be"):
        A.qk_norm_rope_sdpa_nomask(qd, kd, vd, H.dev_bf16(gq)[:D], H.dev_bf16(gk)[:D], eps, None, None, scale, full_row=True)
