"""GPU: a seeded sweep of ragged shapes through the host mirror's entry points (train forward with
Stats, rectangular, key-range mask, key padding, additive mask; both P.V variants; head dims 64, 128,
256; the split schedule forced on and off) and through the backward, each case against the CPU
checker.  Lengths sit on and next to the tile sizes (1, 63..65, 127..129, 255..257, ...).

Bars.  fp16 P.V: max-abs 2e-2 (times V's spread) against the checker's quantized result, Stats 2e-2.
e4m3 P.V: the same, or — rows with only a few keys, where one probability rounded to the other
neighbour moves the output by up to 2^-4 of V's range — an error against fp32 attention no larger
than 1.5 times the checker's own plus 2e-2.  Backward: cosine >= 0.9999 and max-abs 1e-2 of the
largest magnitude, per gradient, against the checker's double-precision backward."""
import numpy as np
import pytest
import torch

from mojodiffusion_amd import _lib
from mojodiffusion_amd import attention_sage as A

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 31, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 511, 640, 700]
KV_LENGTHS = [1, 5, 63, 64, 65, 130, 384, 513, 700]


def _dev(bits):
    return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)


def test_forward_entry_points_over_ragged_shapes(oracle):
    O = oracle
    rng = np.random.default_rng(20240607)
    L = _lib.lib()
    ran = 0
    try:
        for case in range(90):
            D = int(rng.choice([64, 128, 128, 128, 256]))
            B, H = int(rng.integers(1, 3)), int(rng.integers(1, 5))
            Sq = int(rng.choice(LENGTHS))
            kinds = ["plain", "rect", "keymask", "padmask"] + (["addmask"] if D != 256 else [])
            kind = str(rng.choice(kinds))
            Skv = Sq if kind in ("plain", "keymask", "padmask") else int(rng.choice(KV_LENGTHS))
            if kind == "padmask":
                Sq = Skv = int(rng.choice([128, 256, 384, 640]))       # the reference's S_BUF is 128-aligned
            variant = int(rng.integers(0, 2))
            split = int(rng.choice([0, 0, -1, 8, 16, 64, 256]))
            scale = float(1.0 / np.sqrt(D)) * float(rng.choice([1.0, 0.5, 2.0]))
            vstd = float(rng.choice([1.0, 3.0]))
            q = O.f32_to_bf16(rng.standard_normal((B, Sq, H, D)).astype(np.float32))
            koff = rng.standard_normal((B, 1, H, D)) * float(rng.choice([0.0, 2.0, 4.0]))
            k = O.f32_to_bf16((rng.standard_normal((B, Skv, H, D)) + koff).astype(np.float32))
            v = O.f32_to_bf16((rng.standard_normal((B, Skv, H, D)) * vstd).astype(np.float32))
            tag = (case, kind, B, H, Sq, Skv, D, variant, split)
            assert L.mi355_sage_set_attn_split(split) == 0
            qd, kd, vd = _dev(q), _dev(k), _dev(v)
            blkq = 32 if variant == 1 else 128
            stats = want_stats = None
            lo = hi = 0
            addmask = None
            if kind in ("plain", "rect"):
                fwd = (A.sdpa_flash_train_fwd_rect if kind == "rect" else A.sdpa_flash_train_fwd)(qd, kd, vd, scale, variant)
                got, stats = fwd.o, fwd.stats
                _, want, want_stats = O.sdpa_bf16(q, k, v, scale, variant=variant, blkq=blkq, blkk=64, want_stats=True)
            elif kind == "keymask":
                if Skv < 3:
                    continue
                n_txt = int(rng.integers(2, Skv + 1))
                real = int(rng.integers(1, n_txt + 1))
                got = A.sdpa_qwen_keymask(qd, kd, vd, n_txt, real, scale, variant)
                if real < n_txt:
                    lo, hi = real, n_txt
                _, want = O.sdpa_bf16(q, k, v, scale, variant=variant, blkq=blkq, blkk=64, mask_lo=lo, mask_hi=hi)
            elif kind == "padmask":
                real = int(rng.integers(1, Skv + 1))
                got = A.sdpa_flash_fwd_padmask(qd, kd, vd, real, scale, variant).o[:, :real]
                _, want = O.sdpa_bf16(q, k[:, :real], v[:, :real], scale, variant=variant, blkq=blkq, blkk=64)
                want = want[:, :real]
                q, k, v = q[:, :real], k[:, :real], v[:, :real]       # (for the fp32 attention below)
            else:
                mb = O.f32_to_bf16((rng.standard_normal((B, H, Sq, Skv)) * 2.0).astype(np.float32))
                addmask = O.bf16_to_f32(mb)
                got = A.sdpa_cross_masked(qd, kd, vd, _dev(mb), scale, variant)
                _, want = O.sdpa_bf16(q, k, v, scale, variant=variant, blkq=blkq, blkk=64, addmask=addmask)
            torch.cuda.synchronize()
            g = got.float().cpu().numpy()
            assert g.shape == want.shape and np.isfinite(g).all(), tag
            err = float(np.abs(g - want).max())
            if variant == 0:
                assert err <= 2e-2 * vstd, (tag, err)
                if stats is not None:
                    assert float(np.abs(stats.cpu().numpy()[..., 0] - want_stats).max()) <= 2e-2, tag
            elif err > 2e-2 * vstd:
                ref = O.sdpa_f32(O.bf16_to_f32(q), O.bf16_to_f32(k), O.bf16_to_f32(v), scale, mask_lo=lo, mask_hi=hi, addmask=addmask)
                recipe, gerr = float(np.abs(want - ref).max()), float(np.abs(g - ref).max())
                assert gerr <= 1.5 * recipe + 2e-2 * vstd, (tag, err, gerr, recipe)
            ran += 1
    finally:
        L.mi355_sage_set_attn_split(0)
    assert ran >= 80


def test_backward_over_ragged_shapes(oracle):
    O = oracle
    rng = np.random.default_rng(20240608)
    L = _lib.lib()
    for case in range(60):
        D = int(rng.choice([64, 128]))
        B, H = int(rng.integers(1, 3)), int(rng.integers(1, 5))
        Sq = int(rng.choice(LENGTHS[:-1]))
        Skv = Sq if rng.random() < 0.5 else int(rng.choice(KV_LENGTHS[:-1]))
        rq = int(rng.integers(1, Sq + 1)) if rng.random() < 0.4 else 0
        rk = int(rng.integers(1, Skv + 1)) if rng.random() < 0.4 else 0
        spread = float(rng.choice([1.0, 1.0, 2.0]))
        scale = float(1.0 / np.sqrt(D))
        tag = (case, B, H, Sq, Skv, D, rq, rk, spread)
        q, k, v, g = (O.bf16_to_f32(O.f32_to_bf16((rng.standard_normal(s) * spread).astype(np.float32))) for s in
                      ((B, Sq, H, D), (B, Skv, H, D), (B, Skv, H, D), (B, Sq, H, D)))
        nk = rk if 0 < rk < Skv else Skv
        o32, stats = O.sdpa_f32(q, k, v, scale, mask_lo=nk, mask_hi=Skv, want_stats=True)
        o = O.bf16_to_f32(O.f32_to_bf16(o32))
        want = O.sdpa_bwd_f32(q, k, v, g, scale, o=o, stats=stats, real_nq=rq, real_nkv=rk)
        dev = [torch.from_numpy(t).cuda().to(torch.bfloat16) for t in (q, k, v, o, g)]
        st = torch.from_numpy(stats).cuda()
        outs = [torch.full_like(dev[0], 7.0), torch.full_like(dev[1], 7.0), torch.full_like(dev[2], 7.0)]
        ws = torch.empty(L.mi355_sage_bwd_workspace_bytes(B, H, Sq, Skv, D), dtype=torch.uint8, device="cuda")
        qs, ks = _lib.strides_bhnd(Sq, H, D), _lib.strides_bhnd(Skv, H, D)
        rc = L.mi355_sage_sdpa_bwd_bf16(*(t.data_ptr() for t in dev), st.data_ptr(), *(t.data_ptr() for t in outs),
                                        B, H, Sq, Skv, D, scale, qs, ks, ks, qs, qs, qs, ks, ks,
                                        0, 0, 0, 0, 0, 0, 0, 0, 0, 0, rq, rk,
                                        torch.cuda.current_stream().cuda_stream, ws.data_ptr(), ws.numel())
        assert rc == 0, (tag, rc)
        torch.cuda.synchronize()
        for name, got, w in zip(("dQ", "dK", "dV"), outs, want):
            a = got.float().cpu().numpy().astype(np.float64)
            assert np.isfinite(a).all(), (tag, name)
            mag = float(np.abs(w).max())
            # (a gradient that is exactly zero — dK with a single key — comes back as rounding residue)
            assert float(np.abs(a - w).max()) <= 1e-2 * mag + 1e-4, (tag, name)
            if mag > 1e-3:
                b = w.astype(np.float64)
                assert float((a * b).sum() / np.sqrt((a * a).sum() * (b * b).sum())) >= 0.9999, (tag, name)
