"""A gate shaped like the reference's own acceptance test for a new attention backend
(serenitymojo/ops/tests/sdpa_flash_parity.mojo): the trainer shapes, the same generator for the
inputs, agreement with the incumbent, an fp32 referee on the same bf16-rounded values, and speed —
forward, and backward on the saved forward set.  The incumbent here is a bf16 attention with explicit matmuls and an fp32 softmax (what the
reference's math-mode path computes, ops/attention.mojo:332-463); the referee is the same in fp32."""
import time

import numpy as np
import pytest

from mojodiffusion_amd.workloads import f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def _pattern(n, seed, amp):
    """sdpa_flash_parity.mojo:47-55: a 64-bit LCG, top 24 bits -> uniform in [-amp, amp)."""
    out = np.empty(n, np.float32)
    state = np.uint64(seed)
    a, c = np.uint64(6364136223846793005), np.uint64(1442695040888963407)
    # vectorised: state_i = a^i * s0 + c * (a^(i-1) + ... + 1)  computed by doubling
    idx = np.arange(1, n + 1, dtype=np.uint64)
    mul = np.ones(n, np.uint64)
    add = np.zeros(n, np.uint64)
    pa, pc = a, c
    with np.errstate(over="ignore"):
        bit = np.uint64(1)
        while int(bit) <= n:
            sel = (idx & bit) != 0
            mul[sel], add[sel] = mul[sel] * pa, add[sel] * pa + pc
            pa, pc = pa * pa, pc * pa + pc
            bit = bit << np.uint64(1)
        st = mul * state + add
    u = (st >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 16777216.0)
    out[:] = (u * np.float32(2.0) - np.float32(1.0)) * np.float32(amp)
    return out


def test_pattern_generator_matches_a_scalar_loop():
    n = 1000
    want, s = [], 11
    for _ in range(n):
        s = (s * 6364136223846793005 + 1442695040888963407) % (1 << 64)
        want.append((np.float32(s >> 40) * np.float32(1.0 / 16777216.0) * np.float32(2.0) - np.float32(1.0)) * np.float32(1.0))
    np.testing.assert_array_equal(_pattern(n, 11, 1.0), np.array(want, np.float32))


def _agree(a, b):
    a, b = a.double().flatten(), b.double().flatten()
    cos = float((a * b).sum() / (a.norm() * b.norm()))
    return cos, float((a - b).abs().max()), float(((a - b) ** 2).mean().sqrt())


@pytest.mark.parametrize("name,B,S,H,Dh", [("zimage_b1", 1, 1248, 30, 128), ("klein_b1", 1, 1536, 32, 128),
                                           ("zimage_b2", 2, 1248, 30, 128)])
def test_gate_like_the_reference_flash_gate(name, B, S, H, Dh):
    import torch
    import gpu_harness as G
    from mojodiffusion_amd import attention_sage as A
    n = B * S * H * Dh
    scale = 1.0 / np.sqrt(Dh)
    q, k, v = (G.dev_bf16(f32_to_bf16_bits(_pattern(n, seed, 1.0)).reshape(B, S, H, Dh)) for seed in (11, 22, 33))

    def math_mode(q, k, v, dt):
        qh, kh, vh = (x.to(dt).permute(0, 2, 1, 3) for x in (q, k, v))
        s = (qh @ kh.transpose(-1, -2)).float() * scale
        p = torch.softmax(s, dim=-1)
        return (p @ vh.float()).permute(0, 2, 1, 3).to(dt)

    o_math = math_mode(q, k, v, torch.bfloat16)
    o_ref = math_mode(q, k, v, torch.float32)
    o_sage = A.sdpa_nomask(q, k, v, scale)
    torch.cuda.synchronize()
    cos_m, max_m, _ = _agree(o_sage, o_math)
    cos_r, max_r, rms_sage = _agree(o_sage, o_ref)
    _, _, rms_math = _agree(o_math, o_ref)
    print("GATE sdpa_sage %s fwd sage-vs-math cos=%.6f max_abs=%.3e | rms_vs_f32: sage=%.3e math=%.3e"
          % (name, cos_m, max_m, rms_sage, rms_math))
    # 1. same mathematical function as the incumbent (the reference's bar, :154)
    assert cos_m >= 0.999 and cos_r >= 0.999, (cos_m, cos_r)
    assert max_r <= 2e-2, max_r
    # 2. referee, with the reference's own bar (:100-109): not meaningfully worse against fp32 than
    # the bf16 incumbent, rms_err(new) <= 1.5 * rms_err(incumbent) + 1e-7.  (Measured ratio 1.41.)
    assert rms_sage <= 1.5 * rms_math + 1e-7, (rms_sage, rms_math)
    # 3. speed against the incumbent: printed, as the reference's gate prints it; a wall-clock
    # comparison is no pass/fail criterion of a parity test (the measured figures are bench.py's)
    def timeit(fn, reps=5):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps
    t_math = timeit(lambda: math_mode(q, k, v, torch.bfloat16))
    t_sage = timeit(lambda: A.sdpa_nomask(q, k, v, scale))
    print("GATE sdpa_sage %s speed: sage %.3f ms, math-mode %.3f ms" % (name, t_sage * 1e3, t_math * 1e3))

    # ---- backward, as the reference's gate has it (:160-181): d_out from seed 44; the flash
    # backward on the saved forward set against the math-mode backward in bf16 (cos >= 0.999) and,
    # against the fp32 gradients, not worse than 1.5x the bf16 incumbent.  (Measured ratios 0.80-0.96.)
    d_o = G.dev_bf16(f32_to_bf16_bits(_pattern(n, 44, 1.0)).reshape(B, S, H, Dh))

    def math_bwd(dt):
        qq, kk, vv = (x.to(dt).clone().requires_grad_(True) for x in (q, k, v))
        qh, kh, vh = (x.permute(0, 2, 1, 3) for x in (qq, kk, vv))
        p = torch.softmax((qh @ kh.transpose(-1, -2)).float() * scale, dim=-1)
        ((p.to(dt) @ vh).permute(0, 2, 1, 3)).backward(d_o.to(dt))
        return qq.grad, kk.grad, vv.grad

    def sage_fwd_bwd():
        fwd = A.sdpa_flash_train_fwd(q, k, v, scale)
        return A.sdpa_flash_backward(fwd, d_o, scale)

    g_math, g_ref, g = math_bwd(torch.bfloat16), math_bwd(torch.float32), sage_fwd_bwd()
    torch.cuda.synchronize()
    for which, g_sage in (("d_q", g.d_q), ("d_k", g.d_k), ("d_v", g.d_v)):
        i = ("d_q", "d_k", "d_v").index(which)
        cos_m, _, _ = _agree(g_sage, g_math[i])
        _, _, rms_sage = _agree(g_sage, g_ref[i])
        _, _, rms_math = _agree(g_math[i], g_ref[i])
        print("GATE sdpa_sage %s bwd %s sage-vs-math cos=%.6f | rms_vs_f32: sage=%.3e math=%.3e"
              % (name, which, cos_m, rms_sage, rms_math))
        assert cos_m >= 0.999, (which, cos_m)
        assert rms_sage <= 1.5 * rms_math + 1e-7, (which, rms_sage, rms_math)
    t_math = timeit(lambda: math_bwd(torch.bfloat16))
    t_sage = timeit(sage_fwd_bwd)
    print("GATE sdpa_sage %s speed fwd+bwd: sage %.3f ms, math-mode %.3f ms" % (name, t_sage * 1e3, t_math * 1e3))
