"""GPU parity of the attention kernel and the one-shot entry points, through the
C ABI.  Bars: max-abs <= 2e-2 against the CPU checker's quantized attention,
cosine >= 0.999 against the fp32 referee (serenitymojo/parity.mojo:41)."""
import numpy as np
import pytest

from mojodiffusion_amd import _lib
from mojodiffusion_amd.workloads import WORKLOADS, make_inputs, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
COS = 0.999


def _oracle_quantized(oracle, q, k, v, w, variant, mask=(0, 0)):
    import gpu_harness as H
    g = H.oracle_quant_qk(oracle, q, k, w.scale, w.blkq, w.blkk, True, True, mask)
    if variant == 0:
        vq, vs = oracle.quant_v_f16(v, 128, *mask), None
    else:
        vq, vs = oracle.quant_v_fp8(v, 128, *mask)
    return g["q8"], g["qscale"], g["k8"], g["kscale"], vq, vs


@pytest.mark.parametrize("wid,variant,S,mask", [(1, 0, 1024, (0, 0)), (2, 0, 640, (0, 0)), (2, 0, 200, (0, 0)),
                                                (3, 0, 333, (0, 0)), (4, 1, 640, (0, 0)), (2, 1, 200, (0, 0)),
                                                (1, 1, 1024, (0, 0)), (2, 0, 640, (100, 300)), (4, 1, 333, (0, 70)),
                                                (2, 0, 700, (128, 512)), (2, 1, 200, (150, 200))])
def test_attn_kernel_on_checker_quantized_tensors(oracle, wid, variant, S, mask):
    """Feeds the kernel the CPU checker's own quantized tensors, so only the
    attention arithmetic differs.  Masked key ranges start inside, cover whole, and end
    inside 64-key tiles, including the first tile and the ragged last one."""
    import torch
    import gpu_harness as H
    w = WORKLOADS[wid].scaled(B=1, H=2, S=S)
    q, k, v = make_inputs(w)
    q8, qs, k8, ks, vq, vs = _oracle_quantized(oracle, q, k, v, w, variant, mask)
    want16, want32 = oracle.attn(q8, qs, w.blkq, k8, ks, w.blkk, vq, vs, variant, S, S, *mask)
    L = _lib.lib()
    nqp, nkp = L.mi355_sage_pad_q(S), L.mi355_sage_pad_kv(S)
    def padded(x, n, fill):
        out = np.full(x.shape[:2] + (n,) + x.shape[3:], fill, x.dtype)
        out[:, :, :x.shape[2]] = x
        return out
    dq8 = torch.from_numpy(padded(q8, nqp, 0)).cuda()
    dqs = torch.from_numpy(padded(qs, nqp // w.blkq, 1.0)).cuda()
    dk8 = torch.from_numpy(padded(k8, nkp, 0)).cuda()
    dks = torch.from_numpy(padded(ks, nkp // w.blkk, 1.0)).cuda()
    vt = H.tile_v(padded(vq, nkp, 0), variant)
    dv = torch.from_numpy(vt.view(np.int16) if variant == 0 else vt).cuda()
    dvs = torch.from_numpy(vs).cuda() if vs is not None else None
    got, _ = H.attn_fwd(dq8, dqs, w.blkq, dk8, dks, w.blkk, dv, dvs, variant, S, S, mask=mask)
    cos, mx = H.cos_maxabs(bf16_bits_to_f32(got), want32)
    # both variants round every probability to the same significand as the checker (the e4m3
    # variant through its whole-number reference), so they agree far inside the 2e-2 bar
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)


def _one_shot(q, k, v, scale, variant, blkq=None, blkk=64, smooth=True, balance=True):
    import torch
    import gpu_harness as H
    L = _lib.lib()
    B, Sq, Hh, D = q.shape
    Skv = k.shape[1]
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    o = torch.zeros_like(qd)
    qs, ks = _lib.strides_bhnd(Sq, Hh, D), _lib.strides_bhnd(Skv, Hh, D)
    if blkq is None:
        rc = L.mi355_sage_sdpa_bf16(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(), B, Hh, Sq, Skv, D,
                                    scale, qs, ks, ks, qs, 0, 0, 0, 0, 0, H.stream(), variant, None, 0)
    else:
        rc = L.mi355_sage_sdpa_bf16_ex(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(), B, Hh, Sq, Skv, D,
                                       scale, qs, ks, ks, qs, 0, 0, 0, 0, 0, H.stream(), variant, blkq, blkk,
                                       (1 if smooth else 0) | (2 if balance else 0), None, 0)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return H.to_bits(o)


@pytest.mark.parametrize("wid,S", [(1, 1024), (2, 1100), (3, 1100), (4, 1100)])
def test_one_shot_matches_checker_and_referee(oracle, wid, S):
    import gpu_harness as H
    w = WORKLOADS[wid]
    w = w if wid == 1 else w.scaled(B=w.B, H=2, S=S)
    q, k, v = make_inputs(w)
    got = _one_shot(q, k, v, w.scale, w.variant, w.blkq, w.blkk)
    _, want32 = oracle.sdpa_bf16(q, k, v, w.scale, variant=w.variant, blkq=w.blkq, blkk=w.blkk)
    cos, mx = H.cos_maxabs(bf16_bits_to_f32(got), want32)
    assert mx <= MAX_ABS, (cos, mx)
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k), bf16_bits_to_f32(v), w.scale)
    cos_ref, mx_ref = H.cos_maxabs(bf16_bits_to_f32(got), ref)
    assert cos_ref >= COS, (cos_ref, mx_ref)


@pytest.mark.parametrize("wid,S,smooth", [(2, 1100, True), (1, 1024, True), (3, 333, False), (1, 77, True)])
def test_one_shot_equals_stage_pipeline(wid, S, smooth):
    """The one-shot call runs the V passes and the K statistics as roles of one launch and the
    three encoders as roles of another; the stage entry points run subsets of those roles.  The
    stage outputs are proven bit-exact against the CPU checker, so bit-equal O from both routes
    carries that proof over to the one-shot call."""
    import torch
    import gpu_harness as H
    w = WORKLOADS[wid]
    w = w.scaled(B=2, H=3, S=S)
    q, k, v = make_inputs(w)
    got = _one_shot(q, k, v, w.scale, 0, w.blkq, w.blkk, smooth, balance=(wid != 1))
    g = H.quant_qk(q, k, w.scale, w.blkq, w.blkk, smooth, balance=(wid != 1))["dev"]
    gv = H.quant_v(v, 0)["dev"]
    staged, _ = H.attn_fwd(g["q8"], g["qscale"], w.blkq, g["k8"], g["kscale"], w.blkk, gv["vq"], None, 0, S, S)
    np.testing.assert_array_equal(got, staged)


@pytest.mark.parametrize("variant,blkq,D,S", [(0, 128, 128, 700), (0, 64, 128, 333), (1, 32, 128, 520), (0, 32, 64, 1024),
                                               (1, 128, 64, 77)])
def test_attention_stage_that_encodes_q_itself(variant, blkq, D, S):
    """mi355_sage_attn_fwd_q16 (bf16 Q + the stage's channel multipliers) gives the bits of
    mi355_sage_attn_fwd on the stage's q8 / qscale — the kernel's own Q encode is the quantizer's —
    and of the one-shot call, which takes this route; shapes of the split schedule are refused."""
    import gpu_harness as H
    w = WORKLOADS[1 if D == 64 else 2].scaled(B=2, H=3, S=S)
    q, k, v = make_inputs(w)
    g = H.quant_qk(q, k, w.scale, blkq, 64, True)["dev"]
    gv = H.quant_v(v, variant)["dev"]
    staged, _ = H.attn_fwd(g["q8"], g["qscale"], blkq, g["k8"], g["kscale"], 64, gv["vq"], gv["vscale"], variant, S, S)
    rc, fused = H.attn_fwd_q16(q, g["qmul"], blkq, g["k8"], g["kscale"], 64, gv["vq"], gv["vscale"], variant, S)
    assert rc == 0, rc
    np.testing.assert_array_equal(fused, staged)
    np.testing.assert_array_equal(_one_shot(q, k, v, w.scale, variant, blkq, 64), staged)
    big = WORKLOADS[2].scaled(B=1, H=33, S=2048)             # 264 items: the split schedule's
    if _lib.lib().mi355_sage_attn_split_rule(big.B, big.H, big.S, big.S, big.D, 0) > 0:
        qb, kb, vb = make_inputs(big)
        gb = H.quant_qk(qb, kb, big.scale, 128, 64, True)["dev"]
        gvb = H.quant_v(vb, 0)["dev"]
        rc, _ = H.attn_fwd_q16(qb, gb["qmul"], 128, gb["k8"], gb["kscale"], 64, gvb["vq"], None, 0, big.S)
        assert rc == -2, rc


def test_default_recipe_entry_point(oracle):
    """mi355_sage_sdpa_bf16 without the recipe arguments: blkq 128 / blkk 64 / smoothing and balancing on."""
    import gpu_harness as H
    w = WORKLOADS[2].scaled(B=2, H=2, S=384)
    q, k, v = make_inputs(w)
    got = _one_shot(q, k, v, w.scale, 0)
    _, want32 = oracle.sdpa_bf16(q, k, v, w.scale, variant=0, blkq=128, blkk=64)
    cos, mx = H.cos_maxabs(bf16_bits_to_f32(got), want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)


def test_rectangular_and_single_key(oracle):
    import gpu_harness as H
    w = WORKLOADS[2].scaled(B=1, H=2, S=300)
    q, k, v = make_inputs(w)
    got = _one_shot(q[:, :77], k, v, w.scale, 0)
    _, want32 = oracle.sdpa_bf16(q[:, :77], k, v, w.scale)
    cos, mx = H.cos_maxabs(bf16_bits_to_f32(got), want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)
    # one key: softmax is 1 and O is fp16(V) -> bf16, exactly V
    got = _one_shot(q, k[:, :1], v[:, :1], w.scale, 0)
    np.testing.assert_array_equal(got, np.broadcast_to(v[:, :1], got.shape))


def test_properties_constant_v_and_smoothing_invariance(oracle):
    import gpu_harness as H
    w = WORKLOADS[2].scaled(B=1, H=2, S=512)
    q, k, v = make_inputs(w)
    vc = np.ascontiguousarray(np.broadcast_to(v[:, :1], v.shape))
    got = bf16_bits_to_f32(_one_shot(q, k, vc, w.scale, 0))
    np.testing.assert_allclose(got, bf16_bits_to_f32(vc), atol=1.6e-2, rtol=8e-3)
    # shifting every key by one vector changes nothing once K is smoothed (up to the bf16 rounding of K itself)
    shift = np.random.default_rng(3).standard_normal((1, 1, 2, 128)).astype(np.float32) * 8
    k2 = f32_to_bf16_bits(bf16_bits_to_f32(k) + shift)
    a = bf16_bits_to_f32(_one_shot(q, k, v, w.scale, 0))
    b = bf16_bits_to_f32(_one_shot(q, k2, v, w.scale, 0))
    cos, mx = H.cos_maxabs(a, b)
    assert cos >= 0.999, (cos, mx)


def test_sequence_beyond_1024_key_scale_blocks():
    """98 304 keys = 1536 K scale blocks of 64 tokens per head (the kernel stages a head's K scales in
    LDS; up to 4096 of them), one head, e4m3 P.V: sampled rows against an fp32 softmax(QK^T)V, and the
    length one block past the limit is refused."""
    import torch
    L = _lib.lib()
    base = WORKLOADS[5]
    w = base.scaled(B=1, H=1, S=98304)
    q, k, v = _device_inputs(w, 99)
    o = _one_shot_dev(q, k, v, w)
    assert torch.isfinite(o.float()).all()
    g = torch.Generator(device="cuda")
    g.manual_seed(8)
    rows = torch.randint(0, w.S, (256,), generator=g, device="cuda")
    rows[0], rows[1] = 0, w.S - 1
    s = (q[0, rows, 0].float() @ k[0, :, 0].float().T) * w.scale
    ref = torch.softmax(s, dim=-1) @ v[0, :, 0].float()
    got = o[0, rows, 0].float()
    cos = torch.nn.functional.cosine_similarity(got.flatten(), ref.flatten(), dim=0).item()
    assert cos >= COS and (got - ref).abs().max().item() <= 4e-2, (cos, (got - ref).abs().max().item())
    # 4097 scale blocks: refused before anything is launched
    n = 4096 * 64 + 1
    st = _lib.strides_bhnd(n, 1, 128)
    rc = L.mi355_sage_sdpa_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), 1, 1, 256, n, 128, w.scale,
                                _lib.strides_bhnd(256, 1, 128), st, st, _lib.strides_bhnd(256, 1, 128), 0, 0, 0, 0, 0,
                                0, 0, None, 0)
    assert rc == -2


@pytest.mark.parametrize("variant", [0, 1])
def test_reference_maximum_keeps_rising(oracle, variant):
    """Keys grow along the sequence, so the row maximum rises from tile to tile by far more
    than the kernel's lazy-refresh margin: every path that repairs a stale reference
    maximum (refresh + accumulator rescale, redo of an optimistic tile) is exercised, in
    interior tiles, repeatedly.  The second case puts one huge key in the middle.

    Nearly every row here is dominated by one or two keys, and the scores are ~25 times larger
    than on real inputs.  Both variants stay inside the 2e-2 bar on every element: for the e4m3
    variant kernel and checker follow the same rule (whole-number reference, normaliser over the
    rounded probabilities), and with scores this large the kernel forms its exponent arguments
    without the rounding of a large constant, so that a probability next to an e4m3 rounding
    boundary is rounded the way the checker rounds it."""
    import gpu_harness as H
    w = WORKLOADS[2].scaled(B=1, H=2, S=1024, k_offset_std=0.0)
    q, k, v = make_inputs(w)
    kf = bf16_bits_to_f32(k)
    ramp = (1.0 + 24.0 * np.arange(w.S, dtype=np.float32) / w.S)[None, :, None, None]
    k1 = f32_to_bf16_bits(kf * ramp)
    spike = kf.copy()
    spike[:, 517] *= 40.0
    k2 = f32_to_bf16_bits(spike)
    for kk in (k1, k2):
        got = _one_shot(q, kk, v, w.scale, variant, 128, 64, smooth=False)
        _, want32 = oracle.sdpa_bf16(q, kk, v, w.scale, variant=variant, blkq=128, blkk=64, smooth_k=False)
        cos, mx = H.cos_maxabs(bf16_bits_to_f32(got), want32)
        assert cos >= 0.9999, (cos, mx)
        assert mx <= MAX_ABS, (cos, mx)
        assert np.isfinite(bf16_bits_to_f32(got)).all()


@pytest.mark.parametrize("variant", [0, 1])
def test_result_does_not_depend_on_what_ran_before(oracle, variant):
    """Short sequences with an odd and an even number of 64-key tiles (they end in different code of the
    kernel), each computed three times with other work on the device in between that leaves
    different bit patterns in registers, LDS and the library's workspace: the results are the same
    bits every time, and inside the bar against the checker.  (A matrix instruction whose result
    the next instructions did not wait for is the kind of mistake that passes every parity test
    in a fresh process, where the stale contents happen to be the right ones.)"""
    import torch
    import gpu_harness as H
    other = torch.empty(1 << 24, dtype=torch.uint8, device="cuda")
    for S in (192, 256, 320, 448):
        w = WORKLOADS[2].scaled(B=2, H=2, S=S)
        q, k, v = make_inputs(w)
        first = _one_shot(q, k, v, w.scale, variant, w.blkq, w.blkk)
        _, want32 = oracle.sdpa_bf16(q, k, v, w.scale, variant=variant, blkq=w.blkq, blkk=w.blkk)
        cos, mx = H.cos_maxabs(bf16_bits_to_f32(first), want32)
        assert mx <= MAX_ABS and cos >= 0.9999, (S, cos, mx)
        for fill in (0xFF, 0x3C):
            other.fill_(fill)
            big = WORKLOADS[2].scaled(B=1, H=2, S=1024)
            _one_shot(*make_inputs(big), big.scale, 1 - variant)
            other.fill_(fill ^ 0x55)
            torch.cuda.synchronize()
            again = _one_shot(q, k, v, w.scale, variant, w.blkq, w.blkk)
            assert np.array_equal(first, again), (S, fill)


def test_train_fwd_stats_and_padmask(oracle):
    """Stats = natural-log LSE of the scaled scores; real_N_kv masks trailing keys."""
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    w = WORKLOADS[2].scaled(B=1, H=2, S=384)
    q, k, v = make_inputs(w)
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    fwd = A.sdpa_flash_train_fwd(qd, kd, vd, w.scale)
    torch.cuda.synchronize()
    qf, kf, vf = (bf16_bits_to_f32(x).astype(np.float64) for x in (q, k, v))
    s = np.einsum("bihd,bjhd->bhij", qf, kf) * w.scale
    lse = np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1)) + s.max(-1)
    np.testing.assert_allclose(fwd.stats.cpu().numpy()[..., 0], lse, atol=3e-2)
    ref = oracle.sdpa_f32(qf, kf, vf, w.scale)
    cos, mx = H.cos_maxabs(fwd.o.float().cpu().numpy(), ref)
    assert cos >= COS, (cos, mx)
    # key-padding mask: only the first 200 of 384 positions are real
    real = 200
    pm = A.sdpa_flash_fwd_padmask(qd, kd, vd, real, w.scale)
    torch.cuda.synchronize()
    ref = oracle.sdpa_f32(qf[:, :real], kf[:, :real], vf[:, :real], w.scale)
    cos, mx = H.cos_maxabs(pm.o.float().cpu().numpy()[:, :real], ref)
    assert cos >= COS, (cos, mx)


@pytest.mark.parametrize("variant", [0, 1])
def test_stats_rect_f32_and_both_variants(oracle, variant):
    """sdpa_flash_train_fwd_rect (Sq != Skv, with Stats) and sdpa_flash_train_fwd_f32, for the
    fp16 and the e4m3 variant: O against the CPU checker, Stats against the checker's and against
    the log-sum-exp of the fp32 referee."""
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    w = WORKLOADS[2].scaled(B=2, H=2, S=320)
    q, k, v = make_inputs(w)
    q = np.ascontiguousarray(q[:, :200])                               # Sq = 200, Skv = 320
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    fwd = A.sdpa_flash_train_fwd_rect(qd, kd, vd, w.scale, variant)
    torch.cuda.synchronize()
    assert fwd.stats.shape == (w.B, w.H, 200, 1) and fwd.o.shape == qd.shape
    blkq = 128 if variant == 0 else 32
    _, want32, want_stats = oracle.sdpa_bf16(q, k, v, w.scale, variant=variant, blkq=blkq, blkk=64, want_stats=True)
    cos, mx = H.cos_maxabs(fwd.o.float().cpu().numpy(), want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)
    # (e4m3: the normaliser sums rounded probabilities, a few of which round the other way in the checker)
    np.testing.assert_allclose(fwd.stats.cpu().numpy()[..., 0], want_stats, atol=2e-3 if variant == 0 else 1e-2)
    qf, kf, vf = (bf16_bits_to_f32(x) for x in (q, k, v))
    ref, lse = oracle.sdpa_f32(qf, kf, vf, w.scale, want_stats=True)
    np.testing.assert_allclose(fwd.stats.cpu().numpy()[..., 0], lse, atol=3e-2)
    cos, mx = H.cos_maxabs(fwd.o.float().cpu().numpy(), ref)
    assert cos >= COS, (cos, mx)
    # F32 activations: cast to bf16 at the boundary, attend, cast back
    sq = qd[:, :, :, :].float()
    att, fwd32 = A.sdpa_flash_train_fwd_f32(kd.float(), kd.float(), vd.float(), w.scale, variant)
    same = A.sdpa_flash_train_fwd(kd, kd, vd, w.scale, variant)
    torch.cuda.synchronize()
    assert att.dtype == torch.float32 and sq.dtype == torch.float32
    np.testing.assert_array_equal(att.cpu().numpy(), same.o.float().cpu().numpy())
    np.testing.assert_array_equal(fwd32.stats.cpu().numpy(), same.stats.cpu().numpy())


@pytest.mark.parametrize("variant,S,n_txt,real", [(0, 600, 256, 100), (1, 600, 256, 100), (0, 333, 128, 0),
                                                  (0, 520, 200, 200), (1, 450, 450, 77)])
def test_qwen_keymask(oracle, variant, S, n_txt, real):
    """sdpa_qwen_keymask: text keys [real, n_txt) masked, image keys kept.  Against the CPU
    checker with the same mask, against the checker on the tensors with the masked keys removed
    (same result whenever the cut falls on block boundaries; always within the bar), and
    against the fp32 referee.  real == n_txt is no mask at all."""
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    w = WORKLOADS[2].scaled(B=1, H=2, S=S)
    q, k, v = make_inputs(w)
    # what sits in the padded text rows must not matter: make it large
    kx, vx = bf16_bits_to_f32(k), bf16_bits_to_f32(v)
    kx[:, real:n_txt] *= 30.0
    vx[:, real:n_txt] += 100.0
    k, v = f32_to_bf16_bits(kx), f32_to_bf16_bits(vx)
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    got = A.sdpa_qwen_keymask(qd, kd, vd, n_txt, real, w.scale, variant)
    torch.cuda.synchronize()
    gotf = got.float().cpu().numpy()
    blkq = 128 if variant == 0 else 32
    _, want32 = oracle.sdpa_bf16(q, k, v, w.scale, variant=variant, blkq=blkq, blkk=64, mask_lo=real, mask_hi=n_txt)
    cos, mx = H.cos_maxabs(gotf, want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)
    keep = np.r_[0:real, n_txt:S]
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k)[:, keep], bf16_bits_to_f32(v)[:, keep], w.scale)
    cos, mx = H.cos_maxabs(gotf, ref)
    # (few keys make a peaked softmax, where single e4m3 probabilities show)
    assert cos >= COS and mx <= (4e-2 if variant == 0 else 8e-2), (cos, mx)
    if real == n_txt:
        np.testing.assert_array_equal(H.to_bits(got), H.to_bits(A.sdpa_nomask(qd, kd, vd, w.scale, variant)))


@pytest.mark.parametrize("variant", [0, 1])
def test_one_shot_bhsd_memory_and_offsets_for_every_tensor(oracle, variant):
    """Q, K, V and O all in head-major [B,H,S,D] memory at non-zero element offsets inside
    larger buffers, Stats at an offset too: same bits as the plain BSHD call."""
    import ctypes
    import torch
    import gpu_harness as H
    L = _lib.lib()
    w = WORKLOADS[2].scaled(B=2, H=3, S=300)
    q, k, v = make_inputs(w)
    want = _one_shot(q, k, v, w.scale, variant)
    B, S, Hh, D = w.B, w.S, w.H, w.D
    offs = dict(q=64, k=128, v=8, o=200)

    def bhsd_buf(x, off):
        flat = torch.zeros(off + x.size + 64, dtype=torch.bfloat16, device="cuda")
        flat[off:off + x.size] = H.dev_bf16(np.ascontiguousarray(x.transpose(0, 2, 1, 3))).reshape(-1)
        return flat
    qb, kb, vb = bhsd_buf(q, offs["q"]), bhsd_buf(k, offs["k"]), bhsd_buf(v, offs["v"])
    ob = torch.zeros(offs["o"] + q.size + 64, dtype=torch.bfloat16, device="cuda")
    stats = torch.zeros(16 + B * Hh * S, dtype=torch.float32, device="cuda")
    st = (ctypes.c_int64 * 4)(Hh * S * D, S * D, D, 1)
    rc = L.mi355_sage_sdpa_bf16_train_fwd(qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), ob.data_ptr(), stats.data_ptr(),
                                          B, Hh, S, S, D, w.scale, st, st, st, st, offs["q"], offs["k"], offs["v"],
                                          offs["o"], 16, 0, S, S, H.stream(), variant, None, 0)
    assert rc == 0, rc
    torch.cuda.synchronize()
    got = ob[offs["o"]:offs["o"] + q.size].reshape(B, Hh, S, D).permute(0, 2, 1, 3)
    np.testing.assert_array_equal(H.to_bits(got), want)
    assert not ob[:offs["o"]].any() and not ob[offs["o"] + q.size:].any()      # nothing written outside O
    assert not stats[:16].any() and stats[16:].abs().min() > 0
    # rows that are not 16-byte aligned are refused before anything is launched
    assert L.mi355_sage_sdpa_bf16_train_fwd(qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), ob.data_ptr(), stats.data_ptr(),
                                            B, Hh, S, S, D, w.scale, st, st, st, st, offs["q"], offs["k"], 3,
                                            offs["o"], 16, 0, S, S, H.stream(), variant, None, 0) == -2
    bad = (ctypes.c_int64 * 4)(Hh * S * D, S * D, D + 4, 1)
    assert L.mi355_sage_sdpa_bf16_train_fwd(qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), ob.data_ptr(), stats.data_ptr(),
                                            B, Hh, S, S, D, w.scale, st, st, st, bad, offs["q"], offs["k"], offs["v"],
                                            offs["o"], 16, 0, S, S, H.stream(), variant, None, 0) == -2


@pytest.mark.parametrize("variant,Sq,Skv", [(0, 320, 320), (1, 320, 320), (0, 130, 333), (0, 256, 70)])
def test_additive_mask_entry_points(oracle, variant, Sq, Skv):
    """sdpa / sdpa_chunked / sdpa_cross_masked: an additive bias on the scaled scores.  Against
    the CPU checker with the same bias (2e-2) and the biased fp32 referee (cosine 0.999); a -1e4
    block behaves like the key-range mask; a zero bias reproduces the unmasked call;
    a bias broadcast over heads through a zero stride gives the same as its materialised copy."""
    import ctypes
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    w = WORKLOADS[2].scaled(B=2, H=2, S=max(Sq, Skv))
    q, k, v = make_inputs(w)
    q, k, v = np.ascontiguousarray(q[:, :Sq]), np.ascontiguousarray(k[:, :Skv]), np.ascontiguousarray(v[:, :Skv])
    rng = np.random.default_rng(Sq + Skv)
    bias = f32_to_bf16_bits(rng.standard_normal((w.B, w.H, Sq, Skv)).astype(np.float32) * 1.5)
    bias_f = bf16_bits_to_f32(bias)
    bias_f[:, :, :, 5:9] = -np.inf                                   # a few keys removed outright
    bias_f[0, 1, 7, :] = -1e4                                        # one row biased uniformly (cancels)
    bias = f32_to_bf16_bits(np.nan_to_num(bias_f, neginf=-3e38))
    bias_f = bf16_bits_to_f32(bias)
    qd, kd, vd, md = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v), H.dev_bf16(bias)
    fn = A.sdpa if Sq == Skv else A.sdpa_cross_masked
    got = fn(qd, kd, vd, md, w.scale, variant)
    torch.cuda.synchronize()
    gotf = got.float().cpu().numpy()
    blkq = 128 if variant == 0 else 32
    _, want32 = oracle.sdpa_bf16(q, k, v, w.scale, variant=variant, blkq=blkq, blkk=64, addmask=bias_f)
    cos, mx = H.cos_maxabs(gotf, want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k), bf16_bits_to_f32(v), w.scale, addmask=bias_f)
    cos, mx = H.cos_maxabs(gotf, ref)
    assert cos >= COS, (cos, mx)
    if Sq == Skv:
        np.testing.assert_array_equal(H.to_bits(A.sdpa_chunked(qd, kd, vd, md, w.scale, variant)), H.to_bits(got))
        np.testing.assert_array_equal(H.to_bits(A.sdpa_tiled(qd, kd, vd, md, w.scale, variant)), H.to_bits(got))
        with pytest.raises(A.Error, match=r"sdpa_tiled: mask must be \[B,H,S,S\]"):
            A.sdpa_tiled(qd, kd, vd, md[:, :1], w.scale, variant)
        zero = torch.zeros_like(md)
        # (the biased instantiation takes every tile's maximum on the biased scores, the plain one
        # is lazy about it: same function, last-bit differences)
        cz, mz = H.cos_maxabs(A.sdpa(qd, kd, vd, zero, w.scale, variant).float().cpu().numpy(),
                              A.sdpa_nomask(qd, kd, vd, w.scale, variant).float().cpu().numpy())
        assert cz >= 0.99999 and mz <= (4e-3 if variant == 0 else MAX_ABS), (cz, mz)
        # F32 storage: cast at the boundary, result in F32
        o32 = A.sdpa(qd.float(), kd.float(), vd.float(), md.float(), w.scale, variant)
        assert o32.dtype == torch.float32
        np.testing.assert_array_equal(o32.cpu().numpy(), gotf)
    # broadcast over heads through a zero stride, straight through the C ABI
    L = _lib.lib()
    one_head = md[:, :1].contiguous()
    if Skv % 4 == 0:
        ms = (ctypes.c_int64 * 4)(Sq * Skv, 0, Skv, 1)
        o1 = torch.empty_like(qd)
        qs, ks = _lib.strides_bhnd(Sq, w.H, w.D), _lib.strides_bhnd(Skv, w.H, w.D)
        rc = L.mi355_sage_sdpa_bf16_mask(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), one_head.data_ptr(), o1.data_ptr(),
                                         w.B, w.H, Sq, Skv, w.D, w.scale, qs, ks, ks, ms, qs, 0, 0, 0, 0, 0, H.stream(),
                                         variant, None, 0)
        assert rc == 0, rc
        o2 = fn(qd, kd, vd, one_head.expand(-1, w.H, -1, -1).contiguous(), w.scale, variant)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(H.to_bits(o1), H.to_bits(o2))
        bad = (ctypes.c_int64 * 4)(Sq * Skv, 0, Skv + 2, 1)
        assert L.mi355_sage_sdpa_bf16_mask(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), one_head.data_ptr(), o1.data_ptr(),
                                           w.B, w.H, Sq, Skv, w.D, w.scale, qs, ks, ks, bad, qs, 0, 0, 0, 0, 0, H.stream(),
                                           variant, None, 0) == -2


def test_minus_1e4_block_equals_the_key_range_mask(oracle):
    """What sdpa_qwen_keymask does with its -1e4 bias (attention.mojo:804-870), done through the
    additive-mask call: same output as the key-range call to within the quantization of the
    statistics (the range call also keeps the masked keys out of the K statistics)."""
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    w = WORKLOADS[2].scaled(B=1, H=2, S=384)
    q, k, v = (H.dev_bf16(x) for x in make_inputs(w))
    mask = torch.zeros((1, 2, w.S, w.S), dtype=torch.bfloat16, device="cuda")
    mask[..., 100:256] = -1e4
    a = A.sdpa(q, k, v, mask, w.scale)
    b = A.sdpa_qwen_keymask(q, k, v, 256, 100, w.scale)
    torch.cuda.synchronize()
    cos, mx = H.cos_maxabs(a.float().cpu().numpy(), b.float().cpu().numpy())
    assert cos >= 0.9995 and mx <= 3e-2, (cos, mx)


def test_sdpa_nomask_slab_allocates_from_the_slab():
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    w = WORKLOADS[2].scaled(B=1, H=2, S=300)
    q, k, v = (H.dev_bf16(x) for x in make_inputs(w))
    want = A.sdpa_nomask(q, k, v, w.scale)
    slab = A.StepSlab(8 << 20)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    for _ in range(2):
        slab.reset()
        got = A.sdpa_nomask_slab(q, k, v, w.scale, slab)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert got.data_ptr() >= slab.buf.data_ptr() and got.data_ptr() < slab.buf.data_ptr() + slab.capacity_bytes()
    assert slab.n_allocs == 4 and slab.used_bytes() <= slab.peak_bytes() <= slab.capacity_bytes()
    np.testing.assert_array_equal(H.to_bits(got), H.to_bits(want))
    with pytest.raises(A.Error, match="StepSlab: out of space"):
        A.sdpa_nomask_slab(q, k, v, w.scale, A.StepSlab(1 << 16))


def test_internal_workspace_is_per_stream():
    """workspace == NULL on two streams: the calls get separate buffers, so the interleaved
    results equal the single-stream ones bit for bit; growth inside a capture is refused."""
    import torch
    import gpu_harness as H
    L = _lib.lib()
    w = WORKLOADS[2].scaled(B=1, H=2, S=512)
    q, k, v = (H.dev_bf16(x) for x in make_inputs(w))
    q2, k2, v2 = q.flip(1).contiguous(), k.flip(1).contiguous(), v.flip(1).contiguous()
    st = _lib.strides_bhnd(w.S, w.H, w.D)

    def call(qq, kk, vv, out, stream, S=w.S, strides=st):
        return L.mi355_sage_sdpa_bf16(qq.data_ptr(), kk.data_ptr(), vv.data_ptr(), out.data_ptr(), w.B, w.H, S, S, w.D,
                                      w.scale, strides, strides, strides, strides, 0, 0, 0, 0, 0, stream, 0, None, 0)
    ref1, ref2 = torch.empty_like(q), torch.empty_like(q)
    assert call(q, k, v, ref1, H.stream()) == 0 and call(q2, k2, v2, ref2, H.stream()) == 0
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    o1, o2 = torch.empty_like(q), torch.empty_like(q)
    for _ in range(8):
        assert call(q, k, v, o1, s1.cuda_stream) == 0
        assert call(q2, k2, v2, o2, s2.cuda_stream) == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(H.to_bits(o1), H.to_bits(ref1))
    np.testing.assert_array_equal(H.to_bits(o2), H.to_bits(ref2))
    # a stream that is being captured cannot grow its buffer: -3, and the capture stays usable
    s3 = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s3):
        big = torch.zeros((1, 2048, w.H, w.D), dtype=torch.bfloat16, device="cuda")
        obig = torch.empty_like(big)
        stb = _lib.strides_bhnd(2048, w.H, w.D)
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s3):
            rc = call(big, big, big, obig, torch.cuda.current_stream().cuda_stream, 2048, stb)
            obig.zero_()
    assert rc == -3, rc


def test_host_mirror_dtypes_and_workspace_reuse(oracle):
    import torch
    import gpu_harness as H
    from mojodiffusion_amd import attention_sage as A
    w = WORKLOADS[1].scaled(B=1, H=2, S=256)
    q, k, v = make_inputs(w)
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    o1 = A.sdpa_nomask(qd, kd, vd, w.scale)
    o2 = A.sdpa_nomask(qd.float(), kd.float(), vd.float(), w.scale)
    assert o1.dtype == torch.bfloat16 and o2.dtype == torch.float32
    torch.cuda.synchronize()
    np.testing.assert_array_equal(o1.float().cpu().numpy(), o2.cpu().numpy())
    o3 = A.sdpa_nomask_tiled(qd, kd, vd, w.scale)           # same kernel, second call reuses the workspace
    torch.cuda.synchronize()
    np.testing.assert_array_equal(H.to_bits(o1), H.to_bits(o3))
    o4 = A.sdpa_cross_nomask(qd[:, :100].contiguous(), kd, vd, w.scale)
    torch.cuda.synchronize()
    _, want32 = oracle.sdpa_bf16(q[:, :100], k, v, w.scale, blkq=128, blkk=64)
    cos, mx = H.cos_maxabs(o4.float().cpu().numpy(), want32)
    assert mx <= MAX_ABS, (cos, mx)


def test_workload2_full_size(oracle):
    """B=1,H=24,S=4608,D=128: compare two whole Q blocks of three heads with the
    CPU checker (rows are independent), and the whole output with an fp32 SDPA
    computed by torch on the GPU (library referee)."""
    import torch
    import gpu_harness as H
    w = WORKLOADS[2]
    q, k, v = make_inputs(w)
    got = _one_shot(q, k, v, w.scale, 0)
    gotf = bf16_bits_to_f32(got)
    for h in (0, 11, 23):
        for r0 in (0, 4480):
            sl = slice(r0, r0 + 128)
            _, want32 = oracle.sdpa_bf16(q[:, sl, h:h + 1], k[:, :, h:h + 1], v[:, :, h:h + 1], w.scale)
            cos, mx = H.cos_maxabs(gotf[:, sl, h:h + 1], want32)
            assert mx <= MAX_ABS and cos >= 0.9999, (h, r0, cos, mx)
    qd, kd, vd = (H.dev_bf16(x).float().permute(0, 2, 1, 3) for x in (q, k, v))
    ref = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, scale=w.scale).permute(0, 2, 1, 3)
    refn = ref.cpu().numpy()
    cos, mx = H.cos_maxabs(gotf, refn)
    assert cos >= COS, (cos, mx)
    # every row on its own
    num = (gotf.astype(np.float64) * refn).sum(-1)
    den = np.linalg.norm(gotf.astype(np.float64), axis=-1) * np.linalg.norm(refn.astype(np.float64), axis=-1)
    rowcos = num / den
    assert rowcos.min() >= 0.995, rowcos.min()
    assert np.abs(gotf - refn).max() <= 3e-2, np.abs(gotf - refn).max()


def _device_inputs(w, seed):
    from mojodiffusion_amd.workloads import device_inputs
    return device_inputs(w, seed)


def _one_shot_dev(q, k, v, w):
    import torch
    import gpu_harness as H
    L = _lib.lib()
    o = torch.empty_like(q)
    st = _lib.strides_bhnd(w.S, w.H, w.D)
    rc = L.mi355_sage_sdpa_bf16_ex(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), w.B, w.H, w.S, w.S, w.D,
                                   w.scale, st, st, st, st, 0, 0, 0, 0, 0, H.stream(), w.variant, w.blkq, w.blkk,
                                   _lib.K_SMOOTH | _lib.K_BALANCE, None, 0)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return o


@pytest.mark.parametrize("wid", [3, 4, 5])
def test_full_size_properties(wid):
    """Workloads c3 (B2 H30 S4352), c4 (H24 S16896, e4m3 P.V) and c5 (H40 S32760, e4m3 P.V, ragged
    last tile) at their real sizes, through properties that need no full-size referee:
      * sampled query rows against an fp32 softmax(QK^T)V computed with plain matmuls,
      * V constant along the keys: every output row equals that V row,
      * a constant added to every key of a channel (what K smoothing removes) changes nothing
        beyond quantization noise."""
    import torch
    w = WORKLOADS[wid]
    q, k, v = _device_inputs(w, 4242 + wid)
    o = _one_shot_dev(q, k, v, w)
    assert torch.isfinite(o.float()).all()
    # sampled rows of two heads against fp32
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    rows = torch.randint(0, w.S, (192,), generator=g, device="cuda")
    rows[0], rows[1] = 0, w.S - 1
    worst_cos, worst_abs = 1.0, 0.0
    for b, h in ((0, 0), (w.B - 1, w.H - 1)):
        qs = q[b, rows, h].float()
        s = (qs @ k[b, :, h].float().T) * w.scale
        ref = torch.softmax(s, dim=-1) @ v[b, :, h].float()
        got = o[b, rows, h].float()
        cos = torch.nn.functional.cosine_similarity(got.flatten(), ref.flatten(), dim=0).item()
        worst_cos = min(worst_cos, cos)
        worst_abs = max(worst_abs, (got - ref).abs().max().item())
    # Against fp32 (not against the quantized checker) the error is the recipe's own quantization
    # noise, largest for single elements of the e4m3 probabilities of c4/c5 and of c3's outlier
    # channels.
    assert worst_cos >= COS and worst_abs <= 4e-2, (worst_cos, worst_abs)
    # constant V
    vc = v[:, :1].expand(-1, w.S, -1, -1).contiguous()
    oc = _one_shot_dev(q, k, vc, w)
    err = (oc.float() - vc.float()).abs()
    tol = vc.float().abs() * (2.0 ** -7 if w.variant == 0 else 2.0 ** -3) + 1e-6
    assert (err <= tol).all(), err.max().item()
    del vc, oc
    # offset invariance
    off = torch.randn((w.B, 1, w.H, w.D), generator=g, device="cuda") * 2.0
    k2 = (k.float() + off).to(torch.bfloat16)
    o2 = _one_shot_dev(q, k2, v, w)
    cos = torch.nn.functional.cosine_similarity(o.float().flatten(), o2.float().flatten(), dim=0).item()
    assert cos >= 0.999, cos


@pytest.mark.parametrize("variant", [0, 1])
def test_one_shot_call_in_a_hip_graph(variant):
    """With a caller-held workspace the one-shot call allocates nothing and clears its scratch
    with kernels, so it can be captured.  The graph is replayed several times with eager work
    and synchronisations in between and changed inputs; every replay must reproduce the eager
    result of the same inputs bit for bit."""
    import torch
    import gpu_harness as H
    L = _lib.lib()
    w = WORKLOADS[2].scaled(B=1, H=2, S=600)
    q0, k0, v0 = (H.dev_bf16(x) for x in make_inputs(w))
    q, k, v = q0.clone(), k0.clone(), v0.clone()            # static graph inputs
    o = torch.empty_like(q)
    st = _lib.strides_bhnd(w.S, w.H, w.D)
    nws = L.mi355_sage_workspace_bytes(w.B, w.H, w.S, w.S, w.D, variant)
    ws = torch.empty(nws, dtype=torch.uint8, device="cuda")

    def call(out):
        rc = L.mi355_sage_sdpa_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), w.B, w.H, w.S, w.S, w.D,
                                    w.scale, st, st, st, st, 0, 0, 0, 0, 0, torch.cuda.current_stream().cuda_stream,
                                    variant, ws.data_ptr(), nws)
        assert rc == 0, rc

    call(o)                                                  # warm-up outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(o)
    for rep in range(4):
        # new inputs, some unrelated eager work, then the replay
        q.copy_(torch.roll(q0, rep, dims=1))
        k.copy_(k0 * (1.0 + 0.25 * rep))
        v.copy_(torch.roll(v0, -rep, dims=2))
        junk = (q.float() @ q.float().transpose(-1, -2)).sum()
        ws.fill_(0xAB)                                       # the call must not depend on old workspace contents
        torch.cuda.synchronize()
        o.zero_()
        g.replay()
        torch.cuda.synchronize()
        eager = torch.empty_like(o)
        call(eager)
        torch.cuda.synchronize()
        assert torch.isfinite(junk)
        np.testing.assert_array_equal(H.to_bits(o), H.to_bits(eager))
