"""Independent numpy restatement of the quantizers and the quantized attention,
written from the prose rules (not from the C oracle's code) so that the two can
check each other.  numpy's float32 divide is correctly rounded and np.rint is
round-half-to-even, which is what the rules require.

Quantization rules restated:
  per (b,h,d) over the kept keys (a key is kept unless mask_lo <= s < mask_hi):
      mean32 = float32(sum / count) when smoothing, else 0
      s_d    = sqrt(max |f32(k) - mean32|) when balancing (1 if that maximum is 0), else 1
      kmul = 1 / s_d,  qmul = c * s_d,  c = float32(float64(scale) * log2(e))
  Q:  x = f32(bf16) * qmul[b,h,d]
  K:  x = (f32(bf16) - mean32[b,h,d]) * kmul[b,h,d];  masked keys: code 0, not in the block maximum
  per block of `blk` tokens of one (b,h): amax = max|x|; sc = amax/127 (1 if 0);
      code = clip(rint(x / sc), -127, 127)
  V0: fp16(v);  V1: per (b,h,d) amax over tokens; sc = amax/448 (1 if 0); e4m3(v/sc)
"""
import math

import numpy as np
import torch

LOG2E = 1.4426950408889634074


def bf16_to_f32(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


def quant_blocks(x_bhsd, blk, npad_mult, keep=None):
    """x: fp32 [B,H,S,D] already transformed.  Returns codes [B,H,Spad,D], scales [B,H,nblk].
    keep: bool [S]; tokens that are not kept are zeroed first (they then neither raise the block
    maximum nor get a non-zero code)."""
    B, H, S, D = x_bhsd.shape
    if keep is not None:
        x_bhsd = np.where(keep[None, None, :, None], x_bhsd, np.float32(0.0))
    nblk = (S + blk - 1) // blk
    spad = (S + npad_mult - 1) // npad_mult * npad_mult
    codes = np.zeros((B, H, spad, D), np.int8)
    scales = np.zeros((B, H, nblk), np.float32)
    for t in range(nblk):
        tile = x_bhsd[:, :, t * blk:(t + 1) * blk, :]
        amax = np.abs(tile).max(axis=(2, 3)).astype(np.float32)
        sc = np.where(amax > 0, amax / np.float32(127.0), np.float32(1.0)).astype(np.float32)
        c = np.clip(np.rint(tile / sc[:, :, None, None]), -127, 127).astype(np.int8)
        codes[:, :, t * blk:t * blk + tile.shape[2], :] = c
        scales[:, :, t] = sc
    return codes, scales


def quant_q(q_bits_bshd, scale, blkq, npad_mult):
    c = np.float32(np.float64(np.float32(scale)) * LOG2E)
    x = bf16_to_f32(q_bits_bshd).transpose(0, 2, 1, 3) * c
    return quant_blocks(x.astype(np.float32), blkq, npad_mult)


def kmean_exact(k_bits_bshd):
    """Exactly rounded mean: math.fsum is an exact sum."""
    x = bf16_to_f32(k_bits_bshd).transpose(0, 2, 1, 3).astype(np.float64)
    B, H, S, D = x.shape
    mu = np.empty((B, H, D), np.float32)
    for b in range(B):
        for h in range(H):
            for d in range(D):
                mu[b, h, d] = np.float32(math.fsum(x[b, h, :, d]) / S)
    return mu


def kmean_blocked(k_bits_bshd):
    """The normative order: 16-token leaves (ascending), 16-leaf groups, groups ascending."""
    x = bf16_to_f32(k_bits_bshd).transpose(0, 2, 1, 3).astype(np.float64)
    B, H, S, D = x.shape
    total = np.zeros((B, H, D))
    for g0 in range(0, S, 256):
        group = np.zeros((B, H, D))
        for u0 in range(g0, min(S, g0 + 256), 16):
            leaf = np.zeros((B, H, D))
            for s in range(u0, min(S, u0 + 16)):
                leaf = leaf + x[:, :, s, :]
            group = group + leaf
        total = total + group
    return (total / float(S)).astype(np.float32)


def quant_k(k_bits_bshd, mu, blkk, npad_mult, kmul=None, mask_lo=0, mask_hi=0):
    x = bf16_to_f32(k_bits_bshd).transpose(0, 2, 1, 3)
    if mu is not None:
        x = (x - mu[:, :, None, :]).astype(np.float32)
    if kmul is not None:
        x = (x * kmul[:, :, None, :]).astype(np.float32)
    return quant_blocks(x.astype(np.float32), blkk, npad_mult, keep_mask(x.shape[2], mask_lo, mask_hi))


def keep_mask(S, mask_lo, mask_hi):
    s = np.arange(S)
    return ~((s >= mask_lo) & (s < mask_hi))


def quant_q_ch(q_bits_bshd, qmul, blkq, npad_mult):
    x = bf16_to_f32(q_bits_bshd).transpose(0, 2, 1, 3) * qmul[:, :, None, :]
    return quant_blocks(x.astype(np.float32), blkq, npad_mult)


def kstats(k_bits_bshd, scale, smooth, balance, mask_lo=0, mask_hi=0):
    """(mean32, qmul, kmul), each [B,H,D]; the mean is the exactly rounded one (math.fsum)."""
    x = bf16_to_f32(k_bits_bshd).transpose(0, 2, 1, 3)
    B, H, S, D = x.shape
    keep = keep_mask(S, mask_lo, mask_hi)
    xk = x[:, :, keep, :]
    mu = np.zeros((B, H, D), np.float32)
    if smooth:
        x64 = xk.astype(np.float64)
        for b in range(B):
            for h in range(H):
                for d in range(D):
                    mu[b, h, d] = np.float32(math.fsum(x64[b, h, :, d]) / xk.shape[2])
    c = np.float32(np.float64(np.float32(scale)) * LOG2E)
    sd = np.ones((B, H, D), np.float32)
    if balance:
        amax = np.abs((xk - mu[:, :, None, :]).astype(np.float32)).max(axis=2)
        sd = np.where(amax > 0, np.sqrt(amax.astype(np.float32)), np.float32(1.0)).astype(np.float32)
    return mu, (c * sd).astype(np.float32), (np.float32(1.0) / sd).astype(np.float32)


def _pad_tokens(x, npad_mult):
    B, H, S, D = x.shape
    spad = (S + npad_mult - 1) // npad_mult * npad_mult
    out = np.zeros((B, H, spad, D), x.dtype)
    out[:, :, :S] = x
    return out


def quant_v_f16(v_bits_bshd, npad_mult, mask_lo=0, mask_hi=0):
    x = bf16_to_f32(v_bits_bshd).transpose(0, 2, 1, 3)
    x = np.where(keep_mask(x.shape[2], mask_lo, mask_hi)[None, None, :, None], x, np.float32(0.0))
    with np.errstate(over="ignore"):
        h = np.clip(x, -65504.0, 65504.0).astype(np.float16)
    return _pad_tokens(h.view(np.uint16), npad_mult)


def quant_v_fp8(v_bits_bshd, npad_mult, mask_lo=0, mask_hi=0):
    x = bf16_to_f32(v_bits_bshd).transpose(0, 2, 1, 3)
    amax = np.abs(x[:, :, keep_mask(x.shape[2], mask_lo, mask_hi), :]).max(axis=2).astype(np.float32)
    sc = np.where(amax > 0, amax / np.float32(448.0), np.float32(1.0)).astype(np.float32)
    y = (x / sc[:, :, None, :]).astype(np.float32)
    y = np.where(keep_mask(x.shape[2], mask_lo, mask_hi)[None, None, :, None], y, np.float32(0.0))   # masked rows stay 0
    b = torch.from_numpy(np.ascontiguousarray(y)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    return _pad_tokens(b, npad_mult), sc


def attn_float64(q8, qs, blkq, k8, ks, blkk, v_f32, Sq, Skv, p_codec, integer_reference=False,
                 mask_lo=0, mask_hi=0, addmask=None, normalise_by_rounded=False):
    """Quantized attention in float64 from the quantized tensors.
    v_f32: decoded V [B,H,Skv_pad,D] (already multiplied by any per-channel scale).
    p_codec: function rounding p (float32 array in [0,1]) to the P*V operand grid.
    integer_reference: exponentials against ceil(row maximum) instead of the row maximum.
    normalise_by_rounded: divide by the sum of the rounded probabilities instead of the exact ones.
    addmask: [B,H,Sq,Skv] natural-log bias."""
    B, H, _, D = q8.shape
    out = np.zeros((B, Sq, H, D))
    keep = keep_mask(Skv, mask_lo, mask_hi)
    for b in range(B):
        for h in range(H):
            acc = q8[b, h, :Sq].astype(np.int64) @ k8[b, h, :Skv].astype(np.int64).T
            sq = np.repeat(qs[b, h], blkq)[:Sq]
            sk = np.repeat(ks[b, h], blkk)[:Skv]
            s = acc.astype(np.float32) * (sq[:, None] * sk[None, :]).astype(np.float32)
            if addmask is not None:
                s = (s + (addmask[b, h].astype(np.float32) * np.float32(LOG2E)).astype(np.float32)).astype(np.float32)
            s = np.where(keep[None, :], s, np.float32(-np.inf))
            ref = s.max(axis=1, keepdims=True)
            if integer_reference:
                ref = np.ceil(ref)
            p = np.exp2((s - ref).astype(np.float32)).astype(np.float32)
            pr = p_codec(p).astype(np.float64)
            l = (pr if normalise_by_rounded else p.astype(np.float64)).sum(axis=1, keepdims=True)
            out[b, :, h, :] = (pr @ v_f32[b, h, :Skv].astype(np.float64)) / l
    return out


# ---------------------------------------------------------------------------
# RMSNorm + interleaved RoPE in front of the quantizers (bf16 activations)
#   ss   = sum of squares in the order of the reference's kernel (ops/norm.mojo:56-72): a
#          256-slot array holding x[t]^2 (zeros past D) folded in halves, far pairs first
#          (slot t += slot t+128, then +64, ..., +1), fp32 throughout
#   inv  = 1 / sqrt(ss / D + eps)                       (fp32, IEEE)
#   y    = bf16((x * inv) * gain)
#   out[2i], out[2i+1] = bf16(y0*c - y1*s), bf16(y0*s + y1*c)   (products rounded separately)
# ---------------------------------------------------------------------------
def f32_to_bf16_bits_rne(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = u + 0x7FFF + ((u >> 16) & 1)
    return (r >> 16).astype(np.uint16)


def _sumsq_256(x):
    """Sum of squares over the last axis the way a block of 256 threads does it
    (serenitymojo/ops/norm.mojo:56-72): thread t adds x[t]^2, x[t+256]^2, ... in turn, then the
    256 partial sums fold in halves, far pairs first."""
    cols = x.shape[-1]
    part = np.zeros(x.shape[:-1] + (256,), np.float32)
    for c0 in range(0, cols, 256):
        chunk = x[..., c0:c0 + 256]
        part[..., :chunk.shape[-1]] = (part[..., :chunk.shape[-1]] + (chunk * chunk).astype(np.float32)).astype(np.float32)
    while part.shape[-1] > 1:
        half_n = part.shape[-1] // 2
        part = (part[..., :half_n] + part[..., half_n:]).astype(np.float32)
    return part[..., 0]


def norm_rope_bf16(x_bits_bshd, gain_bits, eps, cos=None, sin=None, table_batch_rows=0, halfsplit=False, full_row=False):
    B, S, H, D = x_bits_bshd.shape
    x = bf16_to_f32(x_bits_bshd)                                   # [B,S,H,D]
    if full_row:                                                   # one statistic per token over all H*D channels
        ss = _sumsq_256(x.reshape(B, S, H * D))[..., None]
        mean = (ss / np.float32(H * D)).astype(np.float32)
        g = bf16_to_f32(gain_bits).reshape(H, D)
    else:
        ss = _sumsq_256(x)
        mean = (ss / np.float32(D)).astype(np.float32)
        g = bf16_to_f32(gain_bits)
    inv = (np.float32(1.0) / np.sqrt((mean + np.float32(eps)).astype(np.float32))).astype(np.float32)
    y = ((x * inv[..., None]).astype(np.float32) * g).astype(np.float32)
    y = bf16_to_f32(f32_to_bf16_bits_rne(y))
    if cos is None:
        return f32_to_bf16_bits_rne(y)
    half = D // 2
    rows = (np.arange(B)[:, None, None] * table_batch_rows + np.arange(S)[None, :, None] * H + np.arange(H)[None, None, :])
    tab = (lambda t: bf16_to_f32(np.asarray(t))) if np.asarray(cos).dtype == np.uint16 else (lambda t: np.asarray(t, np.float32))
    c = tab(cos)[rows]                                             # [B,S,H,half]
    s = tab(sin)[rows]
    # pairs (2i, 2i+1), or (i, i + D/2) in the half-split form
    y0, y1 = (y[..., :half], y[..., half:]) if halfsplit else (y[..., 0::2], y[..., 1::2])
    o0 = ((y0 * c).astype(np.float32) - (y1 * s).astype(np.float32)).astype(np.float32)
    o1 = ((y0 * s).astype(np.float32) + (y1 * c).astype(np.float32)).astype(np.float32)
    out = np.empty((B, S, H, D), np.float32)
    if halfsplit:
        out[..., :half], out[..., half:] = o0, o1
    else:
        out[..., 0::2], out[..., 1::2] = o0, o1
    return f32_to_bf16_bits_rne(out)
