"""GPU tests of the 256-channel instantiation (four-wave workgroups, one wave per SIMD): the head
dim of the reference's Ideogram-4 flash arm (serenitymojo/models/dit/ideogram4_dit.mojo:29-49),
forward only as there (ops/tests/sdpa_flash_parity.mojo:212-215).  Same bars as everywhere:
max-abs <= 2e-2 against the CPU checker, cosine >= 0.999 against the fp32 referee."""
import numpy as np
import pytest

from mojodiffusion_amd import _lib
from mojodiffusion_amd.workloads import f32_to_bf16_bits, bf16_bits_to_f32

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
COS = 0.999


def _inputs(B, S, H, D, seed, Skv=None, offset=2.0):
    rng = np.random.default_rng(seed)
    Skv = S if Skv is None else Skv
    q = f32_to_bf16_bits(rng.standard_normal((B, S, H, D)).astype(np.float32))
    k = f32_to_bf16_bits((rng.standard_normal((B, Skv, H, D)) + rng.standard_normal((B, 1, H, D)) * offset).astype(np.float32))
    v = f32_to_bf16_bits(rng.standard_normal((B, Skv, H, D)).astype(np.float32))
    return q, k, v


@pytest.mark.parametrize("variant,B,S,H", [(0, 1, 300, 2), (0, 2, 1153, 3), (1, 1, 300, 2), (1, 2, 1153, 3), (0, 1, 1, 1), (0, 1, 64, 1)])
def test_one_shot_dh256_against_checker_and_referee(oracle, variant, B, S, H):
    import torch
    import gpu_harness as G
    from mojodiffusion_amd import attention_sage as A
    D = 256
    q, k, v = _inputs(B, S, H, D, 100 + S + variant)
    scale = 1.0 / float(np.sqrt(D))
    fwd = A.sdpa_flash_train_fwd(*(G.dev_bf16(x) for x in (q, k, v)), scale, variant)
    torch.cuda.synchronize()
    got = fwd.o.float().cpu().numpy()
    _, want32, want_stats = oracle.sdpa_bf16(q, k, v, scale, variant=variant, blkq=128 if variant == 0 else 32, blkk=64, want_stats=True)
    cos, mx = G.cos_maxabs(got, want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)
    np.testing.assert_allclose(fwd.stats.cpu().numpy()[..., 0], want_stats, atol=2e-3 if variant == 0 else 1e-2)
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k), bf16_bits_to_f32(v), scale)
    cos, mx = G.cos_maxabs(got, ref)
    assert cos >= COS, (cos, mx)
    # same bits through the stage pipeline
    if variant == 0:
        g = G.quant_qk(q, k, scale, 128, 64, True)["dev"]
        gv = G.quant_v(v, 0)["dev"]
        staged, _ = G.attn_fwd(g["q8"], g["qscale"], 128, g["k8"], g["kscale"], 64, gv["vq"], None, 0, S, S)
        np.testing.assert_array_equal(G.to_bits(fwd.o), staged)


def test_dh256_masks_and_rectangular(oracle):
    import torch
    import gpu_harness as G
    from mojodiffusion_amd import attention_sage as A
    B, Sq, Skv, H, D = 1, 200, 333, 2, 256
    q, k, v = _inputs(B, Sq, H, D, 7, Skv=Skv)
    scale = 1.0 / float(np.sqrt(D))
    qd, kd, vd = (G.dev_bf16(x) for x in (q, k, v))
    qf, kf, vf = (bf16_bits_to_f32(x) for x in (q, k, v))
    # rectangular
    got = A.sdpa_cross_nomask(qd, kd, vd, scale).float().cpu().numpy()
    cos, mx = G.cos_maxabs(got, oracle.sdpa_f32(qf, kf, vf, scale))
    assert cos >= COS, (cos, mx)
    # additive mask [B,H,Sq,Skv]
    bias = np.random.default_rng(8).standard_normal((B, H, Sq, Skv)).astype(np.float32)
    bias_d = torch.from_numpy(bias).cuda().to(torch.bfloat16)
    got = A.sdpa_cross_masked(qd, kd, vd, bias_d, scale).float().cpu().numpy()
    s = np.einsum("bihd,bjhd->bhij", qf.astype(np.float64), kf.astype(np.float64)) * scale + bias_d.float().cpu().numpy()
    p = np.exp(s - s.max(-1, keepdims=True))
    ref = np.einsum("bhij,bjhd->bihd", p / p.sum(-1, keepdims=True), vf.astype(np.float64))
    cos, mx = G.cos_maxabs(got, ref)
    assert cos >= COS, (cos, mx)
    # key-range mask (text keys [60, 128) masked) against the checker with the same mask
    got = A.sdpa_qwen_keymask(kd, kd, vd, 128, 60, scale).float().cpu().numpy()
    _, want32 = oracle.sdpa_bf16(k, k, v, scale, variant=0, blkq=128, blkk=64, mask_lo=60, mask_hi=128)
    cos, mx = G.cos_maxabs(got, want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)


def test_dh256_largest_dot_products(oracle):
    """Every Q code +127 and K codes +-127 in all 256 channels: dot = +-4 129 024, more than the
    mantissa room of the accumulator start value the narrower head dims use; this instantiation
    starts its score accumulators at 0.1875 instead.  Half the keys point along q, half against it,
    with different V: the output must be the mean of the aligned half's V."""
    import torch
    import gpu_harness as G
    from mojodiffusion_amd import attention_sage as A
    B, S, H, D = 1, 256, 1, 256
    q = np.full((B, S, H, D), 1.0, np.float32)
    k = np.where((np.arange(S) % 2 == 0)[None, :, None, None], 1.0, -1.0).astype(np.float32) * np.ones((B, S, H, D), np.float32)
    rng = np.random.default_rng(9)
    v = rng.standard_normal((B, S, H, D)).astype(np.float32)
    qb, kb, vb = (f32_to_bf16_bits(x) for x in (q, k, v))
    scale = 1.0 / float(np.sqrt(D))                    # scores +-16: the other half gets exp(-32)
    got = A.sdpa_nomask(*(G.dev_bf16(x) for x in (qb, kb, vb)), scale).float().cpu().numpy()
    assert np.isfinite(got).all()
    want = bf16_bits_to_f32(vb)[:, 0::2].mean(axis=1, keepdims=True)
    np.testing.assert_allclose(got, np.broadcast_to(want, got.shape), atol=4e-3)
    _, want32 = oracle.sdpa_bf16(qb, kb, vb, scale, variant=0, blkq=128, blkk=64)
    cos, mx = G.cos_maxabs(got, want32)
    assert mx <= MAX_ABS, (cos, mx)


def test_dh256_is_forward_only_and_without_fused_pre_ops():
    import ctypes
    import torch
    L = _lib.lib()
    assert L.mi355_sage_workspace_bytes(1, 18, 1153, 1153, 256, 0) > 0
    assert L.mi355_sage_bwd_workspace_bytes(1, 18, 1024, 1024, 256) == 0
    t = torch.zeros((1, 128, 1, 256), dtype=torch.bfloat16, device="cuda")
    st = _lib.strides_bhnd(128, 1, 256)
    stats = torch.zeros((1, 1, 128), dtype=torch.float32, device="cuda")
    p = t.data_ptr()
    rc = L.mi355_sage_sdpa_bwd_bf16(p, p, p, p, p, stats.data_ptr(), p, p, p, 1, 1, 128, 128, 256, 0.1,
                                    st, st, st, st, st, st, st, st, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0,
                                    torch.cuda.current_stream().cuda_stream, None, 0)
    assert rc == -2, rc
    gain = torch.ones(256, dtype=torch.bfloat16, device="cuda")
    rc = L.mi355_sage_sdpa_bf16_norm_rope(p, p, p, p, 1, 1, 128, 128, 256, 0.1, st, st, st, st, 0, 0, 0, 0, 0,
                                          torch.cuda.current_stream().cuda_stream, 0, 128, 64, 3,
                                          gain.data_ptr(), gain.data_ptr(), 1e-6, None, None, 0, 0, None, 0)
    assert rc == -2, rc


@pytest.mark.parametrize("name,B,S,H,Dh", [("ideogram4_fwd_aligned", 1, 1024, 18, 256), ("ideogram4_fwd_pad", 1, 1153, 18, 256)])
def test_gate_fwd_only_cases_of_the_reference_flash_gate(name, B, S, H, Dh):
    """ops/tests/sdpa_flash_parity.mojo:212-275, `_run_fwd_only_case`: seeds 111/222/333, forward
    agreement with the bf16 incumbent (cos >= 0.999), the fp32 referee at the 1.5x rms bar, and
    forward speed."""
    import time
    import torch
    import gpu_harness as G
    from test_gpu_gate import _pattern, _agree
    from mojodiffusion_amd import model_dispatch as M
    n = B * S * H * Dh
    scale = 1.0 / np.sqrt(Dh)
    q, k, v = (G.dev_bf16(f32_to_bf16_bits(_pattern(n, seed, 1.0)).reshape(B, S, H, Dh)) for seed in (111, 222, 333))

    def math_mode(dt):
        qh, kh, vh = (x.to(dt).permute(0, 2, 1, 3) for x in (q, k, v))
        p = torch.softmax((qh @ kh.transpose(-1, -2)).float() * scale, dim=-1)
        return (p @ vh.float()).permute(0, 2, 1, 3).to(dt)

    o_math, o_ref = math_mode(torch.bfloat16), math_mode(torch.float32)
    o_sage = M.ideogram4_sdpa_product_fwd(q, k, v, scale)
    torch.cuda.synchronize()
    cos_m, _, _ = _agree(o_sage, o_math)
    _, _, rms_sage = _agree(o_sage, o_ref)
    _, _, rms_math = _agree(o_math, o_ref)
    print("GATE sdpa_sage %s fwd-only sage-vs-math cos=%.6f | rms_vs_f32: sage=%.3e math=%.3e" % (name, cos_m, rms_sage, rms_math))
    assert cos_m >= 0.999, cos_m
    assert rms_sage <= 1.5 * rms_math + 1e-7, (rms_sage, rms_math)

    def timeit(fn, reps=5):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps
    t_math, t_sage = timeit(lambda: math_mode(torch.bfloat16)), timeit(lambda: M.ideogram4_sdpa_product_fwd(q, k, v, scale))
    print("GATE sdpa_sage %s speed fwd-only: sage %.3f ms, math-mode %.3f ms" % (name, t_sage * 1e3, t_math * 1e3))
    assert t_sage < t_math
