"""The gates of the reference's probe for its memory-efficient SDPA
(serenitymojo/ops/sdpa_tiled_probe.mojo), on the quantized path: the probe's own deterministic
inputs (`_pseudo`, :41-44), shapes and bars (cos >= 0.999, :101, :144, :183), with the fp32 SDPA
as the trusted side where the probe uses its math-mode kernels.

  gate 1   sdpa_nomask_tiled and sdpa_tiled (random additive [B,H,S,S] mask) at S=1536, Dh=128, H=3
  gate 1b  sdpa_cross_nomask (Sq=1536, Skv=1024) against the square call on zero-padded K/V with a
           -1e30 mask on the padded keys
  gate 1c  sdpa_cross_masked with a random [B,H,Sq,Skv] mask against the padded square call
  bf16     the same masked / rectangular calls with BF16 storage at S=64, Dh=64, Skv=48: BF16 out
  gate 2   S=8192 completes with a finite output of the right shape
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

COS = 0.999


def _pseudo(n, salt):
    """sdpa_tiled_probe.mojo:41-44: deterministic values in about [-1, 1]."""
    i = np.arange(n, dtype=np.int64)
    x = (i * 2654435761 + salt * 40503 + 12345) % 100003
    return ((x.astype(np.float32) / np.float32(100003.0)) - np.float32(0.5)) * np.float32(2.0)


def _cos_ratio(a, b):
    a, b = a.double().reshape(-1), b.double().reshape(-1)
    return float(a @ b / (a.norm() * b.norm() + 1e-30)), float(a.norm() / (b.norm() + 1e-30))


def _referee(q, k, v, scale, mask=None):
    """fp32 softmax(q k^T scale + mask) v on [B,S,H,Dh] tensors."""
    import torch
    qq, kk, vv = (t.float().permute(0, 2, 1, 3) for t in (q, k, v))
    s = torch.matmul(qq, kk.transpose(-1, -2)) * scale
    if mask is not None:
        s = s + mask.float()
    return torch.matmul(torch.softmax(s, dim=-1), vv).permute(0, 2, 1, 3)


def _dev(x, shape, dtype):
    import torch
    return torch.from_numpy(x.reshape(shape)).cuda().to(dtype)


@pytest.mark.parametrize("storage", ["f32", "bf16"])
def test_probe_gates(storage):
    import torch
    from mojodiffusion_amd import attention_sage as A
    big = storage == "f32"
    dt = torch.float32 if big else torch.bfloat16
    B, S, H, Dh, Skv = (1, 1536, 3, 128, 1024) if big else (1, 64, 2, 64, 48)
    salts = (1, 2, 3, 7, 17, 19, 23) if big else (31, 32, 33, 34, 35, 36, 37)
    amp_sq, amp_rect = (2.0, 1.5) if big else (1.25, 1.25)
    scale = 1.0 / float(np.sqrt(Dh))
    n = B * S * H * Dh
    q, k, v = (_dev(_pseudo(n, s) * np.float32(0.5), (B, S, H, Dh), dt) for s in salts[:3])

    # gate 1: no mask, and a random additive mask
    got = A.sdpa_nomask_tiled(q, k, v, scale)
    assert got.dtype == dt and got.shape == q.shape
    cos, ratio = _cos_ratio(got, _referee(q, k, v, scale))
    assert cos >= COS and abs(ratio - 1.0) < 2e-2, (cos, ratio)
    mask = _dev(_pseudo(B * H * S * S, salts[3]) * np.float32(amp_sq), (B, H, S, S), dt)
    got = A.sdpa_tiled(q, k, v, mask, scale)
    assert got.dtype == dt
    cos, ratio = _cos_ratio(got, _referee(q, k, v, scale, mask))
    assert cos >= COS and abs(ratio - 1.0) < 2e-2, (cos, ratio)
    np.testing.assert_array_equal(got.float().cpu().numpy(), A.sdpa(q, k, v, mask, scale).float().cpu().numpy())

    # gate 1b: rectangular against the padded square call with the padded keys masked
    ks, vs = (_dev(_pseudo(B * Skv * H * Dh, s) * np.float32(0.5), (B, Skv, H, Dh), dt) for s in salts[4:6])
    k_pad, v_pad = torch.zeros_like(q), torch.zeros_like(q)
    k_pad[:, :Skv], v_pad[:, :Skv] = ks, vs
    cross_mask = torch.zeros((B, H, S, S), dtype=dt, device="cuda")
    cross_mask[..., Skv:] = -1.0e30
    rect = A.sdpa_cross_nomask(q, ks, vs, scale)
    padded = A.sdpa(q, k_pad, v_pad, cross_mask, scale)
    ref = _referee(q, ks, vs, scale)
    for name, t in (("rect", rect), ("padded", padded)):
        assert t.dtype == dt and torch.isfinite(t.float()).all(), name
        cos, ratio = _cos_ratio(t, ref)
        assert cos >= COS and abs(ratio - 1.0) < 2e-2, (name, cos, ratio)
    cos, ratio = _cos_ratio(rect, padded)
    assert cos >= COS, (cos, ratio)

    # gate 1c: masked rectangular against the padded square call
    rect_mask = _dev(_pseudo(B * H * S * Skv, salts[6]) * np.float32(amp_rect), (B, H, S, Skv), dt)
    padded_mask = torch.full((B, H, S, S), -1.0e30, dtype=dt, device="cuda")
    padded_mask[..., :Skv] = rect_mask
    rect_m = A.sdpa_cross_masked(q, ks, vs, rect_mask, scale)
    padded_m = A.sdpa(q, k_pad, v_pad, padded_mask, scale)
    ref = _referee(q, ks, vs, scale, rect_mask)
    assert rect_m.dtype == dt
    for name, t in (("rect", rect_m), ("padded", padded_m)):
        cos, ratio = _cos_ratio(t, ref)
        assert cos >= COS and abs(ratio - 1.0) < 2e-2, (name, cos, ratio)
    cos, ratio = _cos_ratio(rect_m, padded_m)
    assert cos >= COS, (cos, ratio)


def test_probe_gate_2_large_s_completes():
    """S=8192, Dh=128: the math path's [S,S] score slab is what the tiled path exists to avoid."""
    import torch
    from mojodiffusion_amd import attention_sage as A
    B, S, H, Dh = 1, 8192, 4, 128
    n = B * S * H * Dh
    q, k, v = (_dev(_pseudo(n, s) * np.float32(0.5), (B, S, H, Dh), torch.float32) for s in (41, 42, 43))
    got = A.sdpa_nomask_tiled(q, k, v, 1.0 / float(np.sqrt(Dh)))
    torch.cuda.synchronize()
    assert got.shape == (B, S, H, Dh) and got.dtype == torch.float32 and torch.isfinite(got).all()
    cos, ratio = _cos_ratio(got[:, :512], _referee(q[:, :512], k, v, 1.0 / float(np.sqrt(Dh))))
    assert cos >= COS, (cos, ratio)


@pytest.mark.parametrize("Dh", [128, 64])
def test_reviewer_cases_causal_mask_and_fully_masked_row(Dh):
    """The cases of ops/parity/SKEPTIC_FINDINGS_TILED_SDPA_2026-06-03.md: a causal additive mask
    (0 if j <= i else -1e30 — not symmetric, so a transposed mask read fails it), the same with row 0
    masked everywhere (finite large-negative bias: every key ties, the row is the mean of V, no NaN),
    at Dh = 128 and Dh = 64, S = 1536."""
    import torch
    from mojodiffusion_amd import attention_sage as A
    B, S, H = 1, 1536, 3
    scale = 1.0 / float(np.sqrt(Dh))
    n = B * S * H * Dh
    q, k, v = (_dev(_pseudo(n, s) * np.float32(0.5), (B, S, H, Dh), torch.float32) for s in (1, 2, 3))
    i = torch.arange(S, device="cuda")
    causal = torch.where(i[None, :] <= i[:, None], 0.0, -1.0e30).to(torch.float32).expand(B, H, S, S).contiguous()
    got = A.sdpa_tiled(q, k, v, causal, scale)
    assert torch.isfinite(got).all()
    cos, ratio = _cos_ratio(got, _referee(q, k, v, scale, causal))
    assert cos >= COS and abs(ratio - 1.0) < 2e-2, (cos, ratio)
    # the first rows see one, two, three keys: sharp cases of the same check
    np.testing.assert_allclose(got[:, 0].cpu().numpy(), v[:, 0].to(torch.bfloat16).float().cpu().numpy(), atol=4e-3)
    masked_row = causal.clone()
    masked_row[:, :, 0, :] = -1.0e30
    got = A.sdpa_tiled(q, k, v, masked_row, scale)
    assert torch.isfinite(got).all()
    np.testing.assert_allclose(got[:, 0].cpu().numpy(), v.mean(dim=1).cpu().numpy(), atol=2e-3)
    cos, ratio = _cos_ratio(got[:, 1:], _referee(q, k, v, scale, causal)[:, 1:])
    assert cos >= COS, (cos, ratio)


@pytest.mark.parametrize("storage", ["f32", "bf16"])
def test_qwen_keymask_parity_gate(storage):
    """ops/parity/sdpa_qwen_keymask_parity.mojo: the in-kernel mask of the padded text keys
    [real_txt_len, N_TXT) against the full [B,H,S,S] additive mask (-1e4 on those columns), on
    that file's fills ((7i)%17, (5i)%19, (3i)%13), S=7, H=2, N_TXT=4, real_txt_len=2, in F32 and
    BF16 storage, and the case without padding (real_txt_len == N_TXT) against a zero mask.  The
    reference runs it at Dh=8; the kernels here start at Dh=64."""
    import torch
    from mojodiffusion_amd import attention_sage as A
    dt = torch.float32 if storage == "f32" else torch.bfloat16
    B, S, H, Dh, N_TXT = 1, 7, 2, 64, 4
    scale = 1.0 / float(np.sqrt(Dh))
    i = np.arange(B * S * H * Dh, dtype=np.int64)
    q = _dev((((i * 7) % 17).astype(np.float32) - 8.0) * np.float32(0.07), (B, S, H, Dh), dt)
    k = _dev((((i * 5) % 19).astype(np.float32) - 9.0) * np.float32(0.06), (B, S, H, Dh), dt)
    v = _dev((((i * 3) % 13).astype(np.float32) - 6.0) * np.float32(0.05), (B, S, H, Dh), dt)
    for real in (2, N_TXT):
        full_mask = torch.zeros((B, H, S, S), dtype=dt, device="cuda")
        full_mask[..., real:N_TXT] = -1.0e4
        full = A.sdpa(q, k, v, full_mask, scale)
        key = A.sdpa_qwen_keymask(q, k, v, N_TXT, real, scale)
        assert key.dtype == dt and full.dtype == dt
        ref = _referee(q, k, v, scale, full_mask)
        for name, t in (("keymask", key), ("full mask", full)):
            cos, ratio = _cos_ratio(t, ref)
            assert cos >= COS and abs(ratio - 1.0) < 2e-2, (name, real, cos, ratio)
        # serenitymojo/parity.mojo:41-106: cosine >= 0.999 and a max-abs bar between the two paths
        cos, _ = _cos_ratio(key, full)
        assert cos >= 0.9999 and (key.float() - full.float()).abs().max() <= 2e-2, (real, cos)


def test_reference_golden_dh128_through_the_gpu_path():
    """ops/parity/sdpa_math_parity.mojo on the GPU path: the reference's golden output for its
    closed-form inputs at [1,8,32,128] (ops/parity/sdpa_math_ref.txt, tag dh128; H=32 BSHD
    indexing), and `sdpa_nomask` against `sdpa` with a zero mask (:136-237).  F32 storage in, as the
    reference test has it; the bars of the quantized path: cosine >= 0.999, max-abs <= 2e-2."""
    import os
    import torch
    from mojodiffusion_amd import attention_sage as A
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sdpa_math_ref.npz"))["dh128"]
    B, S, H, D = 1, 8, 32, 128
    i = np.arange(B * S * H * D, dtype=np.int64)
    q = _dev((((i * 7) % 13).astype(np.float32) - 6.0) * np.float32(0.05), (B, S, H, D), torch.float32)
    k = _dev((((i * 5) % 11).astype(np.float32) - 5.0) * np.float32(0.05), (B, S, H, D), torch.float32)
    v = _dev((((i * 3) % 9).astype(np.float32) - 4.0) * np.float32(0.05), (B, S, H, D), torch.float32)
    scale = 1.0 / float(np.sqrt(D))
    want = torch.from_numpy(gold.reshape(B, S, H, D)).cuda()
    got = A.sdpa_nomask(q, k, v, scale)
    assert got.dtype == torch.float32
    cos, ratio = _cos_ratio(got, want)
    assert cos >= COS and float((got - want).abs().max()) <= 2e-2, (cos, ratio, float((got - want).abs().max()))
    zero = torch.zeros((B, H, S, S), dtype=torch.float32, device="cuda")
    masked = A.sdpa(q, k, v, zero, scale)
    cos, _ = _cos_ratio(masked, got)
    assert cos >= 0.9999 and float((masked - got).abs().max()) <= 1e-2, cos
    cos, _ = _cos_ratio(masked, want)
    assert cos >= COS, cos
