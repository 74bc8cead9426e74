"""causal = 1 (flame_cudnn_sdpa_bf16's flag, serenitymojo/ops/cshim/cudnn_sdpa.cpp:190-192: cuDNN's
set_causal_mask, query i sees keys j <= i, aligned at the top left for rectangular shapes).  No caller of
the reference's attention path passes it; the kernel honours it by never copying the key tiles past a
workgroup's last row and by masking key > row in the steps on a wave's diagonal.  Checker: the quantized
CPU path given the same mask as an additive bias of -1e4, the way the reference's masked kernels receive
a causal mask (ops/parity/SKEPTIC_FINDINGS_TILED_SDPA_2026-06-03.md); referee: fp32 attention with that bias."""
import numpy as np
import pytest

from mojodiffusion_amd import _lib
from mojodiffusion_amd.workloads import WORKLOADS, make_inputs, bf16_bits_to_f32

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
COS = 0.999


def _bias(B, H, Sq, Skv):
    i, j = np.arange(Sq)[:, None], np.arange(Skv)[None, :]
    return np.broadcast_to(np.where(j <= i, 0.0, -1e4).astype(np.float32), (B, H, Sq, Skv))


def _causal_call(q, k, v, scale, variant, blkq, want_stats=False):
    import torch
    import gpu_harness as H
    L = _lib.lib()
    B, Sq, Hh, D = q.shape
    Skv = k.shape[1]
    qd, kd, vd = H.dev_bf16(q), H.dev_bf16(k), H.dev_bf16(v)
    o = torch.zeros_like(qd)
    qs, ks = _lib.strides_bhnd(Sq, Hh, D), _lib.strides_bhnd(Skv, Hh, D)
    if want_stats:
        stats = torch.zeros((B, Hh, Sq, 1), dtype=torch.float32, device="cuda")
        rc = L.mi355_sage_sdpa_bf16_train_fwd(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(), stats.data_ptr(),
                                              B, Hh, Sq, Skv, D, scale, qs, ks, ks, qs, 0, 0, 0, 0, 0, 1, 0, 0,
                                              H.stream(), variant, None, 0)
    else:
        stats = None
        rc = L.mi355_sage_sdpa_bf16_ex(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(), B, Hh, Sq, Skv, D,
                                       scale, qs, ks, ks, qs, 0, 0, 0, 0, 1, H.stream(), variant, blkq, 64, 3, None, 0)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return H.to_bits(o), (stats.cpu().numpy()[..., 0] if want_stats else None)


@pytest.mark.parametrize("variant,D,Sq,Skv", [(0, 128, 200, 200), (0, 128, 700, 700), (1, 128, 333, 333), (1, 128, 1100, 1100),
                                              (0, 64, 1024, 1024), (0, 128, 300, 520), (0, 128, 520, 300), (1, 128, 257, 64),
                                              (0, 256, 300, 300), (0, 128, 1, 77), (0, 128, 2304, 2304)])
def test_causal_against_the_checker_and_the_referee(oracle, variant, D, Sq, Skv):
    import gpu_harness as H
    w = WORKLOADS[1 if D == 64 else 2].scaled(B=1, H=2, S=max(Sq, Skv), D=D)
    q, k, v = make_inputs(w)
    q, k, v = q[:, :Sq], k[:, :Skv], v[:, :Skv]
    blkq = 128 if variant == 0 else 32
    got, _ = _causal_call(q, k, v, w.scale, variant, blkq)
    bias = _bias(1, 2, Sq, Skv)
    _, want32 = oracle.sdpa_bf16(q, k, v, w.scale, variant=variant, blkq=blkq, blkk=64, addmask=bias)
    cos, mx = H.cos_maxabs(bf16_bits_to_f32(got), want32)
    assert mx <= MAX_ABS and cos >= 0.9999, (cos, mx)
    ref = oracle.sdpa_f32(bf16_bits_to_f32(q), bf16_bits_to_f32(k), bf16_bits_to_f32(v), w.scale, addmask=bias)
    cos_ref, mx_ref = H.cos_maxabs(bf16_bits_to_f32(got), ref)
    assert cos_ref >= COS, (cos_ref, mx_ref)
    # the first row sees key 0 only: its output is V[0], to the quantization of V (fp16: exact on bf16
    # inputs in range; e4m3: three mantissa bits under a per-channel scale)
    v0 = bf16_bits_to_f32(v)[:, 0]
    assert np.abs(bf16_bits_to_f32(got)[:, 0] - v0).max() <= MAX_ABS + (0.0 if variant == 0 else 0.07) * np.abs(v0).max()


def test_causal_stats_and_no_effect_of_later_keys(oracle):
    """With Stats: the log-sum-exp over the keys a row sees.  And the property that defines the mask:
    changing K and V rows after position p changes nothing in the output rows up to p (the K statistics
    are kept equal by changing the rows in a way that preserves every channel's sum, minimum and maximum:
    a permutation of those rows)."""
    import gpu_harness as H
    w = WORKLOADS[2].scaled(B=1, H=2, S=640)
    q, k, v = make_inputs(w)
    got, stats = _causal_call(q, k, v, w.scale, 0, 128, want_stats=True)
    qf, kf = (bf16_bits_to_f32(x).astype(np.float64) for x in (q, k))
    s = np.einsum("bihd,bjhd->bhij", qf, kf) * w.scale + _bias(1, 2, w.S, w.S)
    lse = np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1)) + s.max(-1)
    np.testing.assert_allclose(stats, lse, atol=3e-2)
    p = 300
    perm = np.concatenate([np.arange(p + 1), p + 1 + np.random.default_rng(3).permutation(w.S - p - 1)])
    got2, _ = _causal_call(q, k[:, perm], v[:, perm], w.scale, 0, 128, want_stats=True)
    np.testing.assert_array_equal(got[:, :p + 1 - 64], got2[:, :p + 1 - 64])
