"""ctypes binding of the CPU oracle (oracle/libsage_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg as the checker.  The product package
(mojodiffusion_amd) never imports this module.

All tensors are numpy arrays; bf16 / fp16 tensors are carried as uint16 bit
patterns, e4m3 as uint8.  Tensors are addressed as logical [B, H, N, D] via
element strides, so a [B, S, H, Dh] array is passed with strides_bshd(...).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsage_oracle.so")
_lib = None

_i64p = ctypes.POINTER(ctypes.c_int64)


def build(force=False):
    """Compile the oracle with the Makefile next to this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.sage_oracle_bf16_to_f32.restype = ctypes.c_float
        L.sage_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.sage_oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.sage_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.sage_oracle_f16_to_f32.restype = ctypes.c_float
        L.sage_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.sage_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.sage_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.sage_oracle_e4m3_to_f32.restype = ctypes.c_float
        L.sage_oracle_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.sage_oracle_f32_to_e4m3.restype = ctypes.c_uint8
        L.sage_oracle_f32_to_e4m3.argtypes = [ctypes.c_float]
        L.sage_oracle_pad.restype = ctypes.c_int64
        L.sage_oracle_pad.argtypes = [ctypes.c_int64, ctypes.c_int64]
        for name in ("sage_oracle_f32_to_bf16_n", "sage_oracle_f32_to_f16_n",
                     "sage_oracle_f32_to_e4m3_n", "sage_oracle_e4m3_to_f32_n"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
        for name in ("sage_oracle_sdpa_f32", "sage_oracle_sdpa_online_f32"):
            getattr(L, name).restype = ctypes.c_int
            getattr(L, name).argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 5 + [ctypes.c_float] + [_i64p] * 4
        L.sage_oracle_quant_q.restype = ctypes.c_int
        L.sage_oracle_quant_q.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_float,
                                          ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        L.sage_oracle_sdpa_f32_ex.restype = ctypes.c_int
        L.sage_oracle_sdpa_f32_ex.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [
                                              ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        L.sage_oracle_sdpa_bwd_f32.restype = ctypes.c_int
        L.sage_oracle_sdpa_bwd_f32.argtypes = [ctypes.c_void_p] * 9 + [ctypes.c_int] * 5 + [ctypes.c_float] + [_i64p] * 8 + [
                                               ctypes.c_int, ctypes.c_int]
        L.sage_oracle_kstats.restype = ctypes.c_int
        L.sage_oracle_kstats.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_float] + [ctypes.c_int] * 3 + [
                                         ctypes.c_void_p] * 3
        L.sage_oracle_quant_q_ch.restype = ctypes.c_int
        L.sage_oracle_quant_q_ch.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_float, ctypes.c_void_p,
                                             ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        L.sage_oracle_quant_k_ch.restype = ctypes.c_int
        L.sage_oracle_quant_k_ch.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_void_p, ctypes.c_void_p] + [
                                             ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.c_void_p]
        L.sage_oracle_quant_v_f16_masked.restype = ctypes.c_int
        L.sage_oracle_quant_v_f16_masked.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p] + [ctypes.c_int] * 3 + [
                                                     ctypes.c_void_p]
        L.sage_oracle_quant_v_fp8_masked.restype = ctypes.c_int
        L.sage_oracle_quant_v_fp8_masked.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p] + [ctypes.c_int] * 3 + [
                                                     ctypes.c_void_p, ctypes.c_void_p]
        L.sage_oracle_attn_ex.restype = ctypes.c_int
        L.sage_oracle_attn_ex.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
                                          ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
                                          ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int] + [ctypes.c_int] * 5 + [
                                          ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                          ctypes.c_void_p, ctypes.c_void_p, _i64p, ctypes.c_void_p]
        L.sage_oracle_sdpa_bf16_ex.restype = ctypes.c_int
        L.sage_oracle_sdpa_bf16_ex.argtypes = [ctypes.c_void_p] * 6 + [ctypes.c_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [
                                               ctypes.c_int] * 6 + [ctypes.c_void_p]
        L.sage_oracle_kmean.restype = ctypes.c_int
        L.sage_oracle_kmean.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_void_p]
        L.sage_oracle_quant_k.restype = ctypes.c_int
        L.sage_oracle_quant_k.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_void_p,
                                          ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        L.sage_oracle_quant_v_f16.restype = ctypes.c_int
        L.sage_oracle_quant_v_f16.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_int, ctypes.c_void_p]
        L.sage_oracle_quant_v_fp8.restype = ctypes.c_int
        L.sage_oracle_quant_v_fp8.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_int,
                                              ctypes.c_void_p, ctypes.c_void_p]
        L.sage_oracle_attn.restype = ctypes.c_int
        L.sage_oracle_attn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
                                       ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
                                       ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int] + [ctypes.c_int] * 5 + [
                                       ctypes.c_void_p, ctypes.c_void_p, _i64p]
        L.sage_oracle_sdpa_bf16.restype = ctypes.c_int
        L.sage_oracle_sdpa_bf16.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [
                                            ctypes.c_int] * 4
        L.sage_oracle_rms_norm_f32.restype = ctypes.c_int
        L.sage_oracle_rms_norm_f32.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
                                               ctypes.c_float, ctypes.c_void_p]
        L.sage_oracle_rope_interleaved_f32.restype = ctypes.c_int
        L.sage_oracle_rope_interleaved_f32.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        L.sage_oracle_rope_halfsplit_f32.restype = ctypes.c_int
        L.sage_oracle_rope_halfsplit_f32.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        L.sage_oracle_norm_rope_bf16_ex.restype = ctypes.c_int
        L.sage_oracle_norm_rope_bf16_ex.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_void_p, ctypes.c_float,
                                                    ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        L.sage_oracle_norm_rope_bf16.restype = ctypes.c_int
        L.sage_oracle_norm_rope_bf16.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 4 + [_i64p, ctypes.c_void_p, ctypes.c_float,
                                                 ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        L.sage_oracle_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


# ---------------------------------------------------------------------------
# layout helpers
# ---------------------------------------------------------------------------

def strides_bshd(S, H, D):
    """[B,S,H,D] contiguous memory seen as logical [B,H,N,D]
    (serenitymojo/ops/attention_flash.mojo:46-54)."""
    return (ctypes.c_int64 * 4)(S * H * D, D, H * D, 1)


def strides_bhsd(H, S, D):
    return (ctypes.c_int64 * 4)(H * S * D, S * D, D, 1)


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _chk(rc, what):
    if rc != 0:
        raise RuntimeError("%s: oracle rc=%d" % (what, rc))


def pad(n, mult):
    return (n + mult - 1) // mult * mult


# ---------------------------------------------------------------------------
# codecs (vector forms)
# ---------------------------------------------------------------------------

def f32_to_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, np.uint16)
    lib().sage_oracle_f32_to_bf16_n(_p(x), _p(y), x.size)
    return y


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_f16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, np.uint16)
    lib().sage_oracle_f32_to_f16_n(_p(x), _p(y), x.size)
    return y


def f32_to_e4m3(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, np.uint8)
    lib().sage_oracle_f32_to_e4m3_n(_p(x), _p(y), x.size)
    return y


def e4m3_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint8)
    y = np.empty(b.shape, np.float32)
    lib().sage_oracle_e4m3_to_f32_n(_p(b), _p(y), b.size)
    return y


# ---------------------------------------------------------------------------
# SDPA on [B,S,H,D] arrays (the reference's physical layout)
# ---------------------------------------------------------------------------

def _dims_bshd(q, k):
    B, Sq, H, D = q.shape
    Skv = k.shape[1]
    return B, H, Sq, Skv, D


def sdpa_f32(q, k, v, scale, online=False, mask_lo=0, mask_hi=0, addmask=None, want_stats=False):
    """fp32 inputs [B,S,H,D] -> fp32 output [B,Sq,H,D].  Keys [mask_lo, mask_hi) are left out;
    addmask: additive bias [B,H,Sq,Skv] fp32 (natural-log units); want_stats: also return the
    log-sum-exp [B,H,Sq]."""
    q, k, v = (np.ascontiguousarray(t, dtype=np.float32) for t in (q, k, v))
    B, H, Sq, Skv, D = _dims_bshd(q, k)
    o = np.empty_like(q)
    args = (_p(q), _p(k), _p(v), _p(o), B, H, Sq, Skv, D, scale,
            strides_bshd(Sq, H, D), strides_bshd(Skv, H, D), strides_bshd(Skv, H, D), strides_bshd(Sq, H, D))
    if online:
        assert mask_hi <= mask_lo and addmask is None and not want_stats
        _chk(lib().sage_oracle_sdpa_online_f32(*args), "sdpa_online_f32")
        return o
    if addmask is not None:
        addmask = np.ascontiguousarray(addmask, dtype=np.float32)
        assert addmask.shape == (B, H, Sq, Skv)
    stats = np.empty((B, H, Sq), np.float32) if want_stats else None
    _chk(lib().sage_oracle_sdpa_f32_ex(*args, mask_lo, mask_hi, _p(addmask), _p(stats)), "sdpa_f32")
    return (o, stats) if want_stats else o


def sdpa_bwd_f32(q, k, v, dout, scale, o=None, stats=None, real_nq=0, real_nkv=0):
    """Gradients (dq, dk, dv), fp32 [B,S,H,D], of softmax(q k^T * scale) v against the upstream
    gradient dout.  With o [B,Sq,H,D] and stats [B,H,Sq] given, the flash form: probabilities from
    the caller's log-sum-exp, row term rowsum(dout * o).  real_nq / real_nkv: valid lengths."""
    q, k, v, dout = (np.ascontiguousarray(t, dtype=np.float32) for t in (q, k, v, dout))
    B, H, Sq, Skv, D = _dims_bshd(q, k)
    assert (o is None) == (stats is None)
    if o is not None:
        o = np.ascontiguousarray(o, dtype=np.float32)
        stats = np.ascontiguousarray(stats, dtype=np.float32)
        assert o.shape == q.shape and stats.shape == (B, H, Sq)
    dq, dk, dv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    sq, sk = strides_bshd(Sq, H, D), strides_bshd(Skv, H, D)
    _chk(lib().sage_oracle_sdpa_bwd_f32(_p(q), _p(k), _p(v), _p(o), _p(dout), _p(stats), _p(dq), _p(dk), _p(dv),
                                        B, H, Sq, Skv, D, scale, sq, sk, sk, sq, sq, sq, sk, sk,
                                        real_nq, real_nkv), "sdpa_bwd_f32")
    return dq, dk, dv


def rms_norm_f32(x, g, eps):
    """x [rows, cols] fp32, g [cols] fp32 -> fp32 (serenitymojo/ops/norm.mojo:47-79)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    g = np.ascontiguousarray(g, dtype=np.float32)
    out = np.empty_like(x)
    _chk(lib().sage_oracle_rms_norm_f32(_p(x), _p(g), x.shape[0], x.shape[1], eps, _p(out)), "rms_norm_f32")
    return out


def rope_interleaved_f32(x, cos, sin):
    """x [rows, D], cos/sin [rows, D/2], all fp32 (serenitymojo/ops/rope.mojo:7-9)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    cos = np.ascontiguousarray(cos, dtype=np.float32)
    sin = np.ascontiguousarray(sin, dtype=np.float32)
    if cos.shape != (x.shape[0], x.shape[1] // 2) or sin.shape != cos.shape:
        raise ValueError("rope_interleaved_f32: cos/sin must be [rows, D/2] with one row per row of x")
    out = np.empty_like(x)
    _chk(lib().sage_oracle_rope_interleaved_f32(_p(x), _p(cos), _p(sin), x.shape[0], x.shape[1], _p(out)),
         "rope_interleaved_f32")
    return out


def rope_halfsplit_f32(x, cos, sin):
    """x [rows, D], cos/sin [rows, D/2], all fp32; pairs (x[i], x[i + D/2]) (serenitymojo/ops/rope.mojo:10-13)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    cos = np.ascontiguousarray(cos, dtype=np.float32)
    sin = np.ascontiguousarray(sin, dtype=np.float32)
    if cos.shape != (x.shape[0], x.shape[1] // 2) or sin.shape != cos.shape:
        raise ValueError("rope_halfsplit_f32: cos/sin must be [rows, D/2] with one row per row of x")
    out = np.empty_like(x)
    _chk(lib().sage_oracle_rope_halfsplit_f32(_p(x), _p(cos), _p(sin), x.shape[0], x.shape[1], _p(out)),
         "rope_halfsplit_f32")
    return out


PRE_HALFSPLIT = 1
PRE_TABLES_BF16 = 2
PRE_NORM_FULL_ROW = 4


def norm_rope_bf16(x_bf16, gain_bf16, eps, cos=None, sin=None, table_batch_rows=0, halfsplit=False, full_row=False):
    """x: uint16 [B,S,H,D] bf16 bits; gain: uint16 [D] (or [H*D] with full_row: the RMSNorm then
    runs over all H*D channels of a token); cos/sin: fp32, or uint16 bf16 bits, [rows, D/2] with row
    s*H + h (plus b*table_batch_rows), or None for no rotation; halfsplit: pairs (i, i + D/2)
    instead of (2i, 2i+1).  Returns uint16 [B,S,H,D]."""
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    g = np.ascontiguousarray(gain_bf16, dtype=np.uint16)
    B, S, H, D = x.shape
    y = np.empty_like(x)
    flags = (PRE_HALFSPLIT if halfsplit else 0) | (PRE_NORM_FULL_ROW if full_row else 0)
    if cos is not None:
        if np.asarray(cos).dtype == np.uint16:
            flags |= PRE_TABLES_BF16
            cos = np.ascontiguousarray(cos, dtype=np.uint16)
            sin = np.ascontiguousarray(sin, dtype=np.uint16)
        else:
            cos = np.ascontiguousarray(cos, dtype=np.float32)
            sin = np.ascontiguousarray(sin, dtype=np.float32)
        need = (B - 1) * table_batch_rows + S * H
        if cos.shape[0] < need or cos.shape[1] != D // 2 or sin.shape != cos.shape:
            raise ValueError("norm_rope_bf16: cos/sin must be [>= %d, %d]" % (need, D // 2))
    if g.shape != ((H * D,) if full_row else (D,)):
        raise ValueError("norm_rope_bf16: gain must be [%d]" % (H * D if full_row else D))
    _chk(lib().sage_oracle_norm_rope_bf16_ex(_p(x), B, H, S, D, strides_bshd(S, H, D), _p(g), eps,
                                             _p(cos) if cos is not None else None,
                                             _p(sin) if sin is not None else None, table_batch_rows,
                                             flags, _p(y)),
         "norm_rope_bf16")
    return y


def quant_q(q_bf16, scale, blkq, npad_mult=None):
    """q_bf16: uint16 [B,S,H,D].  Returns (q8 [B,H,Spad,D] int8, qscale [B,H,nblk] f32)."""
    q = np.ascontiguousarray(q_bf16, dtype=np.uint16)
    B, S, H, D = q.shape
    mult = npad_mult or blkq
    q8 = np.empty((B, H, pad(S, mult), D), np.int8)
    sc = np.empty((B, H, (S + blkq - 1) // blkq), np.float32)
    _chk(lib().sage_oracle_quant_q(_p(q), B, H, S, D, strides_bshd(S, H, D), scale, blkq, mult,
                                   _p(q8), _p(sc)), "quant_q")
    return q8, sc


def kstats(k_bf16, scale, flags, mask_lo=0, mask_hi=0):
    """Per-channel K statistics.  Returns (kmean, qmul, kmul), each [B,H,D] fp32."""
    k = np.ascontiguousarray(k_bf16, dtype=np.uint16)
    B, S, H, D = k.shape
    mu, qm, km = (np.empty((B, H, D), np.float32) for _ in range(3))
    _chk(lib().sage_oracle_kstats(_p(k), B, H, S, D, strides_bshd(S, H, D), scale, flags, mask_lo, mask_hi,
                                  _p(mu), _p(qm), _p(km)), "kstats")
    return mu, qm, km


def quant_q_ch(q_bf16, scale, qmul, blkq, npad_mult=None):
    """Q with a per-channel multiplier qmul [B,H,D] (None: the scalar c)."""
    q = np.ascontiguousarray(q_bf16, dtype=np.uint16)
    B, S, H, D = q.shape
    mult = npad_mult or blkq
    q8 = np.empty((B, H, pad(S, mult), D), np.int8)
    sc = np.empty((B, H, (S + blkq - 1) // blkq), np.float32)
    if qmul is not None:
        qmul = np.ascontiguousarray(qmul, dtype=np.float32)
    _chk(lib().sage_oracle_quant_q_ch(_p(q), B, H, S, D, strides_bshd(S, H, D), scale, _p(qmul), blkq, mult,
                                      _p(q8), _p(sc)), "quant_q_ch")
    return q8, sc


def quant_k_ch(k_bf16, mu, kmul, blkk, npad_mult=None, mask_lo=0, mask_hi=0):
    k = np.ascontiguousarray(k_bf16, dtype=np.uint16)
    B, S, H, D = k.shape
    mult = npad_mult or blkk
    k8 = np.empty((B, H, pad(S, mult), D), np.int8)
    sc = np.empty((B, H, (S + blkk - 1) // blkk), np.float32)
    mu = None if mu is None else np.ascontiguousarray(mu, dtype=np.float32)
    kmul = None if kmul is None else np.ascontiguousarray(kmul, dtype=np.float32)
    _chk(lib().sage_oracle_quant_k_ch(_p(k), B, H, S, D, strides_bshd(S, H, D), _p(mu), _p(kmul),
                                      mask_lo, mask_hi, blkk, mult, _p(k8), _p(sc)), "quant_k_ch")
    return k8, sc


def kmean(k_bf16):
    k = np.ascontiguousarray(k_bf16, dtype=np.uint16)
    B, S, H, D = k.shape
    mu = np.empty((B, H, D), np.float32)
    _chk(lib().sage_oracle_kmean(_p(k), B, H, S, D, strides_bshd(S, H, D), _p(mu)), "kmean")
    return mu


def quant_k(k_bf16, mu, blkk, npad_mult=None):
    k = np.ascontiguousarray(k_bf16, dtype=np.uint16)
    B, S, H, D = k.shape
    mult = npad_mult or blkk
    k8 = np.empty((B, H, pad(S, mult), D), np.int8)
    sc = np.empty((B, H, (S + blkk - 1) // blkk), np.float32)
    if mu is not None:
        mu = np.ascontiguousarray(mu, dtype=np.float32)
    _chk(lib().sage_oracle_quant_k(_p(k), B, H, S, D, strides_bshd(S, H, D), _p(mu), blkk, mult,
                                   _p(k8), _p(sc)), "quant_k")
    return k8, sc


def quant_v_f16(v_bf16, npad_mult, mask_lo=0, mask_hi=0):
    v = np.ascontiguousarray(v_bf16, dtype=np.uint16)
    B, S, H, D = v.shape
    v16 = np.empty((B, H, pad(S, npad_mult), D), np.uint16)
    _chk(lib().sage_oracle_quant_v_f16_masked(_p(v), B, H, S, D, strides_bshd(S, H, D), mask_lo, mask_hi,
                                              npad_mult, _p(v16)), "quant_v_f16")
    return v16


def quant_v_fp8(v_bf16, npad_mult, mask_lo=0, mask_hi=0):
    v = np.ascontiguousarray(v_bf16, dtype=np.uint16)
    B, S, H, D = v.shape
    v8 = np.empty((B, H, pad(S, npad_mult), D), np.uint8)
    vs = np.empty((B, H, D), np.float32)
    _chk(lib().sage_oracle_quant_v_fp8_masked(_p(v), B, H, S, D, strides_bshd(S, H, D), mask_lo, mask_hi,
                                              npad_mult, _p(v8), _p(vs)), "quant_v_fp8")
    return v8, vs


def attn(q8, qscale, blkq, k8, kscale, blkk, vq, vscale, variant, Sq, Skv, mask_lo=0, mask_hi=0,
         addmask=None, qshift=None, want_stats=False):
    """Quantized tensors in the oracle's plain [B,H,Npad,D] layout.
    Returns (o_bf16 uint16 [B,Sq,H,D], o_f32 [B,Sq,H,D]) and, with want_stats, stats [B,H,Sq]."""
    B, H, NqPad, D = q8.shape
    NkvPad = k8.shape[2]
    o16 = np.empty((B, Sq, H, D), np.uint16)
    o32 = np.empty((B, Sq, H, D), np.float32)
    if addmask is not None:
        addmask = np.ascontiguousarray(addmask, dtype=np.float32)
        assert addmask.shape == (B, H, Sq, Skv)
    if qshift is not None:
        qshift = np.ascontiguousarray(qshift, dtype=np.float32)
        assert qshift.shape == (B, H, NqPad)
    stats = np.empty((B, H, Sq), np.float32) if want_stats else None
    _chk(lib().sage_oracle_attn_ex(_p(q8), _p(qscale), blkq, NqPad, _p(k8), _p(kscale), blkk, NkvPad,
                                   _p(vq), _p(vscale), variant, B, H, Sq, Skv, D, mask_lo, mask_hi,
                                   _p(addmask), _p(qshift), _p(o16), _p(o32), strides_bshd(Sq, H, D), _p(stats)), "attn")
    return (o16, o32, stats) if want_stats else (o16, o32)


K_SMOOTH = 1
K_BALANCE = 2


def sdpa_bf16(q, k, v, scale, variant=0, blkq=128, blkk=64, smooth_k=True, balance=True,
              mask_lo=0, mask_hi=0, addmask=None, want_stats=False):
    """Whole quantized path on bf16 (uint16) [B,S,H,D] inputs.
    Returns (o_bf16 uint16, o_f32) and, with want_stats, stats [B,H,Sq]."""
    q, k, v = (np.ascontiguousarray(t, dtype=np.uint16) for t in (q, k, v))
    B, H, Sq, Skv, D = _dims_bshd(q, k)
    o16 = np.empty((B, Sq, H, D), np.uint16)
    o32 = np.empty((B, Sq, H, D), np.float32)
    if addmask is not None:
        addmask = np.ascontiguousarray(addmask, dtype=np.float32)
        assert addmask.shape == (B, H, Sq, Skv)
    stats = np.empty((B, H, Sq), np.float32) if want_stats else None
    flags = (K_SMOOTH if smooth_k else 0) | (K_BALANCE if balance else 0)
    _chk(lib().sage_oracle_sdpa_bf16_ex(_p(q), _p(k), _p(v), _p(o16), _p(o32), _p(stats), B, H, Sq, Skv, D, scale,
                                        strides_bshd(Sq, H, D), strides_bshd(Skv, H, D),
                                        strides_bshd(Skv, H, D), strides_bshd(Sq, H, D),
                                        variant, blkq, blkk, flags, mask_lo, mask_hi, _p(addmask)), "sdpa_bf16")
    return (o16, o32, stats) if want_stats else (o16, o32)


def num_threads():
    return lib().sage_oracle_num_threads()
