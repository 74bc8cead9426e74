"""Helpers for the GPU parity tests: calls the stage entry points of
libmi355_sage.so through ctypes on torch-owned device buffers and brings the
results back as numpy arrays in the CPU checker's plain layouts."""
import ctypes

import numpy as np
import torch

from mojodiffusion_amd import _lib


def dev_bf16(bits_u16):
    """uint16 bf16 bit patterns (numpy) -> bf16 cuda tensor of the same shape."""
    return torch.from_numpy(bits_u16.view(np.int16)).cuda().view(torch.bfloat16)


def to_bits(t):
    """bf16 cuda tensor -> uint16 numpy bit patterns."""
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def stream():
    return torch.cuda.current_stream().cuda_stream


def v_slots(variant):
    L = _lib.lib()
    return np.array([L.mi355_sage_v_slot(k, variant) for k in range(64)])


def untile_v(vt, variant):
    """[B,H,T,D,64 slots] -> plain [B,H,T*64,D]."""
    slots = v_slots(variant)
    B, H, T, D, _ = vt.shape
    return np.ascontiguousarray(vt[..., slots].transpose(0, 1, 2, 4, 3)).reshape(B, H, T * 64, D)


def tile_v(v_plain, variant):
    """plain [B,H,Npad,D] (Npad % 64 == 0) -> [B,H,T,D,64 slots]."""
    slots = v_slots(variant)
    B, H, N, D = v_plain.shape
    x = v_plain.reshape(B, H, N // 64, 64, D).transpose(0, 1, 2, 4, 3)      # [B,H,T,D,key]
    out = np.empty_like(x)
    out[..., slots] = x
    return np.ascontiguousarray(out)


def quant_qk(q_bits, k_bits, scale, blkq, blkk, smooth_k, strides_q=None, strides_k=None,
             q_off=0, k_off=0, shape=None, balance=True, mask=(0, 0)):
    """q_bits/k_bits: uint16 [B,S,H,D] (or any buffer when shape/strides are given).
    Returns dict of numpy arrays in the padded device layouts."""
    L = _lib.lib()
    if shape is None:
        B, Sq, H, D = q_bits.shape
        Skv = k_bits.shape[1]
        strides_q = _lib.strides_bhnd(Sq, H, D)
        strides_k = _lib.strides_bhnd(Skv, H, D)
    else:
        B, H, Sq, Skv, D = shape
    qd, kd = dev_bf16(q_bits), dev_bf16(k_bits)
    nqp, nkp = L.mi355_sage_pad_q(Sq), L.mi355_sage_pad_kv(Skv)
    q8 = torch.full((B, H, nqp, D), 77, dtype=torch.int8, device="cuda")
    k8 = torch.full((B, H, nkp, D), 77, dtype=torch.int8, device="cuda")
    qs = torch.full((B, H, nqp // blkq), -1.0, dtype=torch.float32, device="cuda")
    ks = torch.full((B, H, nkp // blkk), -1.0, dtype=torch.float32, device="cuda")
    km, qm, kmu = (torch.full((B, H, D), -1.0, dtype=torch.float32, device="cuda") for _ in range(3))
    nscr = L.mi355_sage_quant_scratch_bytes(B, H, Skv, D)
    scr = torch.full((max(nscr, 8),), 0xAB, dtype=torch.uint8, device="cuda")
    flags = (_lib.K_SMOOTH if smooth_k else 0) | (_lib.K_BALANCE if balance else 0)
    rc = L.mi355_sage_quant_qk_bf16(qd.data_ptr(), kd.data_ptr(), B, H, Sq, Skv, D, scale,
                                    strides_q, strides_k, q_off, k_off, blkq, blkk, flags, mask[0], mask[1],
                                    q8.data_ptr(), qs.data_ptr(), k8.data_ptr(), ks.data_ptr(),
                                    km.data_ptr(), qm.data_ptr(), kmu.data_ptr(), scr.data_ptr(), scr.numel(), stream())
    assert rc == 0, rc
    torch.cuda.synchronize()
    return dict(q8=q8.cpu().numpy(), qscale=qs.cpu().numpy(), k8=k8.cpu().numpy(), kscale=ks.cpu().numpy(),
                kmean=km.cpu().numpy(), qmul=qm.cpu().numpy(), kmul=kmu.cpu().numpy(),
                dev=dict(q8=q8, qscale=qs, k8=k8, kscale=ks, kmean=km, qmul=qm, kmul=kmu))


def oracle_quant_qk(oracle, q_bits, k_bits, scale, blkq, blkk, smooth_k=True, balance=True, mask=(0, 0)):
    """The CPU checker's statistics and codes in the device's padded layouts."""
    L = _lib.lib()
    flags = (1 if smooth_k else 0) | (2 if balance else 0)
    mu, qmul, kmul = oracle.kstats(k_bits, scale, flags, *mask)
    q8, qs = oracle.quant_q_ch(q_bits, scale, qmul, blkq, int(L.mi355_sage_pad_q(1)))
    k8, ks = oracle.quant_k_ch(k_bits, mu, kmul, blkk, 128, *mask)
    return dict(q8=q8, qscale=qs, k8=k8, kscale=ks, kmean=mu, qmul=qmul, kmul=kmul)


def quant_v(v_bits, variant, mask=(0, 0), strides=None, v_off=0, shape=None):
    L = _lib.lib()
    if shape is None:
        B, S, H, D = v_bits.shape
        st = _lib.strides_bhnd(S, H, D)
    else:
        B, H, S, D = shape
        st = strides
    vd = dev_bf16(v_bits)
    nkp = L.mi355_sage_pad_kv(S)
    if variant == 0:
        out = torch.full((B, H, nkp // 64, D, 64), 0x7E00, dtype=torch.int16, device="cuda")
        rc = L.mi355_sage_quant_v_f16(vd.data_ptr(), B, H, S, D, st, v_off, mask[0], mask[1], out.data_ptr(), stream())
        assert rc == 0, rc
        torch.cuda.synchronize()
        return dict(vq=out.cpu().numpy().view(np.uint16), vscale=None, dev=dict(vq=out, vscale=None))
    out = torch.full((B, H, nkp // 64, D, 64), 0x7F, dtype=torch.uint8, device="cuda")
    vs = torch.full((B, H, D), -1.0, dtype=torch.float32, device="cuda")
    nscr = L.mi355_sage_quant_scratch_bytes(B, H, S, D)
    scr = torch.full((max(nscr, 8),), 0xAB, dtype=torch.uint8, device="cuda")
    rc = L.mi355_sage_quant_v_fp8(vd.data_ptr(), B, H, S, D, st, v_off, mask[0], mask[1], out.data_ptr(), vs.data_ptr(),
                                  scr.data_ptr(), scr.numel(), stream())
    assert rc == 0, rc
    torch.cuda.synchronize()
    return dict(vq=out.cpu().numpy(), vscale=vs.cpu().numpy(), dev=dict(vq=out, vscale=vs))


def quant_qkv(q_bits, k_bits, v_bits, scale, variant, blkq, blkk, mask=(0, 0), encode_q=True):
    """mi355_sage_quant_qkv_bf16: the three launches of the one-shot calls.  Same dict as quant_qk plus vq, vscale.
    encode_q False: q8 and qscale are passed as NULL (Q is left to mi355_sage_attn_fwd_q16)."""
    L = _lib.lib()
    B, Sq, H, D = q_bits.shape
    Skv = k_bits.shape[1]
    sq, sk = _lib.strides_bhnd(Sq, H, D), _lib.strides_bhnd(Skv, H, D)
    qd, kd, vd = dev_bf16(q_bits), dev_bf16(k_bits), dev_bf16(v_bits)
    nqp, nkp = L.mi355_sage_pad_q(Sq), L.mi355_sage_pad_kv(Skv)
    q8 = torch.full((B, H, nqp, D), 77, dtype=torch.int8, device="cuda")
    k8 = torch.full((B, H, nkp, D), 77, dtype=torch.int8, device="cuda")
    qs = torch.full((B, H, nqp // blkq), -1.0, dtype=torch.float32, device="cuda")
    ks = torch.full((B, H, nkp // blkk), -1.0, dtype=torch.float32, device="cuda")
    km, qm, kmu, vs = (torch.full((B, H, D), -1.0, dtype=torch.float32, device="cuda") for _ in range(4))
    vq = torch.full((B, H, nkp // 64, D, 64), 0x7E, dtype=torch.int16 if variant == 0 else torch.uint8, device="cuda")
    scr = torch.full((max(L.mi355_sage_quant_scratch_bytes(B, H, Skv, D), 8),), 0xAB, dtype=torch.uint8, device="cuda")
    rc = L.mi355_sage_quant_qkv_bf16(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), B, H, Sq, Skv, D, scale, sq, sk, sk, 0, 0, 0,
                                     variant, blkq, blkk, _lib.K_SMOOTH | _lib.K_BALANCE, mask[0], mask[1],
                                     q8.data_ptr() if encode_q else None, qs.data_ptr() if encode_q else None, k8.data_ptr(),
                                     ks.data_ptr(), km.data_ptr(), qm.data_ptr(),
                                     kmu.data_ptr(), vq.data_ptr(), vs.data_ptr(), scr.data_ptr(), scr.numel(), stream())
    assert rc == 0, rc
    torch.cuda.synchronize()
    vq_np = vq.cpu().numpy()
    return dict(q8=q8.cpu().numpy(), qscale=qs.cpu().numpy(), k8=k8.cpu().numpy(), kscale=ks.cpu().numpy(),
                kmean=km.cpu().numpy(), qmul=qm.cpu().numpy(), kmul=kmu.cpu().numpy(),
                vq=vq_np.view(np.uint16) if variant == 0 else vq_np, vscale=vs.cpu().numpy() if variant == 1 else None)


def attn_fwd(q8, qscale, blkq, k8, kscale, blkk, vq, vscale, variant, Sq, Skv, kv_valid=None, want_stats=False,
             mask=(0, 0), qshift=None):
    """Device tensors in the device layouts.  Returns (o bits uint16 [B,Sq,H,D], stats or None)."""
    L = _lib.lib()
    B, H, _, D = q8.shape
    o = torch.zeros((B, Sq, H, D), dtype=torch.bfloat16, device="cuda")
    stats = torch.zeros((B, H, Sq), dtype=torch.float32, device="cuda") if want_stats else None
    rc = L.mi355_sage_attn_fwd(q8.data_ptr(), qscale.data_ptr(), blkq, k8.data_ptr(), kscale.data_ptr(), blkk,
                               vq.data_ptr(), vscale.data_ptr() if vscale is not None else None, variant,
                               B, H, Sq, Skv, kv_valid or Skv, mask[0], mask[1], D, o.data_ptr(),
                               _lib.strides_bhnd(Sq, H, D), 0, qshift.data_ptr() if qshift is not None else None,
                               stats.data_ptr() if want_stats else None, stream())
    assert rc == 0, rc
    torch.cuda.synchronize()
    return to_bits(o), (stats.cpu().numpy() if want_stats else None)


def attn_fwd_q16(q_bits, qmul, blkq, k8, kscale, blkk, vq, vscale, variant, Skv, kv_valid=None, mask=(0, 0)):
    """mi355_sage_attn_fwd_q16: Q as bf16 bits [B,Sq,H,D] (host), the other operands as device tensors.
    Returns the return code and O bits."""
    L = _lib.lib()
    B, Sq, H, D = q_bits.shape
    qd = dev_bf16(q_bits)
    o = torch.zeros((B, Sq, H, D), dtype=torch.bfloat16, device="cuda")
    st = _lib.strides_bhnd(Sq, H, D)
    rc = L.mi355_sage_attn_fwd_q16(qd.data_ptr(), st, 0, qmul.data_ptr(), blkq, k8.data_ptr(), kscale.data_ptr(), blkk,
                                   vq.data_ptr(), vscale.data_ptr() if vscale is not None else None, variant,
                                   B, H, Sq, Skv, kv_valid or Skv, mask[0], mask[1], D, o.data_ptr(), st, 0, stream())
    torch.cuda.synchronize()
    return rc, to_bits(o)


def cos_maxabs(a, b):
    """serenitymojo/parity.mojo:57-93 (float64 cosine + max-abs)."""
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    den = np.sqrt((a * a).sum()) * np.sqrt((b * b).sum())
    cos = 1.0 if den == 0 else float((a * b).sum() / den)
    return cos, float(np.abs(a - b).max())
