"""GPU tests of the per-model dispatch arms (mojodiffusion_amd/model_dispatch.py): dtype flow of
the reference's `*_sdpa_product_fwd` functions and of krea2's three attention paths, against the
direct calls (same bits) and the fp32 referee."""
import numpy as np
import pytest

from mojodiffusion_amd.workloads import WORKLOADS, make_inputs, bf16_bits_to_f32

pytestmark = pytest.mark.gpu

COS = 0.999


def _inputs(wid, B, H, S):
    import gpu_harness as Hh
    w = WORKLOADS[wid].scaled(B=B, H=H, S=S)
    q, k, v = make_inputs(w)
    return w, (q, k, v), tuple(Hh.dev_bf16(x) for x in (q, k, v))


def test_product_fwd_arms_bf16_and_f32(oracle):
    import torch
    import gpu_harness as Hh
    from mojodiffusion_amd import attention_sage as A, model_dispatch as M
    w, (q, k, v), (qd, kd, vd) = _inputs(3, 1, 3, 333)
    want = A.sdpa_flash_train_fwd(qd, kd, vd, w.scale).o
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k), bf16_bits_to_f32(v), w.scale)
    for fn in (M.zimage_sdpa_product_fwd, M.ltx2_sdpa_product_fwd):
        got = fn(qd, kd, vd, w.scale)
        assert got.dtype == torch.bfloat16 and got.shape == qd.shape
        np.testing.assert_array_equal(Hh.to_bits(got), Hh.to_bits(want))
        # F32 in -> cast at the boundary -> F32 out, the same values
        got32 = fn(qd.float(), kd.float(), vd.float(), w.scale)
        assert got32.dtype == torch.float32
        np.testing.assert_array_equal(got32.cpu().numpy(), want.float().cpu().numpy())
        cos, mx = Hh.cos_maxabs(got32.cpu().numpy(), ref)
        assert cos >= COS, (cos, mx)
    # rectangular arm (LTX-2 cross attention)
    qs = qd[:, :200].contiguous()
    got = M.ltx2_sdpa_product_fwd_rect(qs.float(), kd.float(), vd.float(), w.scale)
    np.testing.assert_array_equal(got.cpu().numpy(), A.sdpa_flash_train_fwd_rect(qs, kd, vd, w.scale).o.float().cpu().numpy())
    # the Ideogram-4 arm (Dh = 256 in that model) is the same function
    np.testing.assert_array_equal(Hh.to_bits(M.ideogram4_sdpa_product_fwd(qd, kd, vd, w.scale)), Hh.to_bits(want))
    # a head dim the library does not cover: no silent fallback
    with pytest.raises(A.Error):
        M.zimage_sdpa_product_fwd(qd[..., :96].contiguous(), kd[..., :96].contiguous(), vd[..., :96].contiguous(), w.scale)
    # a switched-off arm fails loudly too
    M.ZIMAGE_SDPA_SAGE = False
    try:
        with pytest.raises(A.Error):
            M.zimage_sdpa_product_fwd(qd, kd, vd, w.scale)
    finally:
        M.ZIMAGE_SDPA_SAGE = True


def test_krea2_three_paths(oracle):
    """real_len -> trailing keys masked; additive mask; neither.  F32 in, F32 out, scale 1/sqrt(Dh)."""
    import torch
    import gpu_harness as Hh
    from mojodiffusion_amd import attention_sage as A, model_dispatch as M
    w, (q, k, v), (qd, kd, vd) = _inputs(2, 1, 4, 384)
    q32, k32, v32 = qd.float(), kd.float(), vd.float()
    scale = 1.0 / np.sqrt(w.D)
    qf, kf, vf = (bf16_bits_to_f32(x) for x in (q, k, v))
    # (c) no mask
    got = M.krea2_attention_sdpa(q32, k32, v32)
    assert got.dtype == torch.float32
    np.testing.assert_array_equal(got.cpu().numpy(), A.sdpa_nomask_tiled(qd, kd, vd, scale).float().cpu().numpy())
    cos, mx = Hh.cos_maxabs(got.cpu().numpy(), oracle.sdpa_f32(qf, kf, vf, scale))
    assert cos >= COS, (cos, mx)
    # (a) real_len
    real = 300
    got = M.krea2_attention_sdpa(q32, k32, v32, real_len=real)
    cos, mx = Hh.cos_maxabs(got.cpu().numpy()[:, :real], oracle.sdpa_f32(qf[:, :real], kf[:, :real], vf[:, :real], scale))
    assert cos >= COS, (cos, mx)
    # (b) additive pad mask: -1e4 on the same trailing keys gives the same attention on the real rows
    mask = torch.zeros((1, w.H, w.S, w.S), dtype=torch.float32, device="cuda")
    mask[..., real:] = -1.0e4
    got_b = M.krea2_attention_sdpa(q32, k32, v32, mask=mask)
    assert got_b.dtype == torch.float32
    cos, mx = Hh.cos_maxabs(got_b.cpu().numpy()[:, :real], oracle.sdpa_f32(qf[:, :real], kf[:, :real], vf[:, :real], scale))
    assert cos >= COS, (cos, mx)


def test_klein_train_fwd_keeps_the_backward_set():
    import torch
    import gpu_harness as Hh
    from mojodiffusion_amd import attention_sage as A, model_dispatch as M
    w, _, (qd, kd, vd) = _inputs(2, 1, 2, 384)
    att, fwd = M.klein_sdpa_train_fwd(qd.float(), kd.float(), vd.float(), w.scale)
    assert att.dtype == torch.float32 and fwd.o.dtype == torch.bfloat16 and fwd.stats.shape == (1, w.H, w.S, 1)
    g = torch.randn_like(att)
    grads = A.sdpa_flash_backward_f32(fwd.q_pad, fwd.k_pad, fwd.v_pad, fwd.o, fwd.stats, g, w.scale)
    torch.cuda.synchronize()
    for t in (grads.d_q, grads.d_k, grads.d_v):
        assert t.dtype == torch.float32 and torch.isfinite(t).all() and t.abs().max() > 0
