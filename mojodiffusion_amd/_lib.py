"""ctypes loader for libmi355_sage.so.  There is no fallback: if the library is
missing, every attention call fails with an error that says how to build it."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmi355_sage.so")

_i64p = ctypes.POINTER(ctypes.c_int64)
_vp = ctypes.c_void_p
_int = ctypes.c_int
_i64 = ctypes.c_int64

# name -> (restype, argtypes); mirrors include/mi355_sage.h one to one
SIGNATURES = {
    "mi355_sage_sdpa_bf16": (_int, [_vp] * 4 + [_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [_i64] * 4
                             + [_int, _vp, _int, _vp, ctypes.c_size_t]),
    "mi355_sage_sdpa_bf16_static": (_int, [_vp] * 4 + [_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [_i64] * 4
                                    + [_int, _vp, _int]),
    "mi355_sage_static_scratch_bytes": (ctypes.c_size_t, []),
    "mi355_sage_sdpa_bf16_ex": (_int, [_vp] * 4 + [_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [_i64] * 4
                                + [_int, _vp, _int, _int, _int, _int, _vp, ctypes.c_size_t]),
    "mi355_sage_sdpa_bf16_train_fwd": (_int, [_vp] * 5 + [_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [_i64] * 5
                                       + [_int, _int, _int, _vp, _int, _vp, ctypes.c_size_t]),
    "mi355_sage_sdpa_bf16_keymask": (_int, [_vp] * 5 + [_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [_i64] * 5
                                     + [_int, _int, _vp, _int, _vp, ctypes.c_size_t]),
    "mi355_sage_sdpa_bf16_mask": (_int, [_vp] * 5 + [_int] * 5 + [ctypes.c_float] + [_i64p] * 5 + [_i64] * 5
                                  + [_vp, _int, _vp, ctypes.c_size_t]),
    "mi355_sage_workspace_bytes": (ctypes.c_size_t, [_int] * 6),
    "mi355_sage_bwd_workspace_bytes": (ctypes.c_size_t, [_int] * 5),
    "mi355_sage_sdpa_bwd_bf16": (_int, [_vp] * 9 + [_int] * 5 + [ctypes.c_float] + [_i64p] * 8 + [_i64] * 9
                                 + [_int, _int, _int, _vp, _vp, ctypes.c_size_t]),
    "mi355_sage_pad_q": (_i64, [_i64]),
    "mi355_sage_pad_kv": (_i64, [_i64]),
    "mi355_sage_v_slot": (_int, [_int, _int]),
    "mi355_sage_quant_scratch_bytes": (ctypes.c_size_t, [_int] * 4),
    "mi355_sage_quant_qk_bf16": (_int, [_vp, _vp] + [_int] * 5 + [ctypes.c_float, _i64p, _i64p, _i64, _i64]
                                 + [_int] * 5 + [_vp] * 8 + [ctypes.c_size_t, _vp]),
    "mi355_sage_quant_qkv_bf16": (_int, [_vp] * 3 + [_int] * 5 + [ctypes.c_float, _i64p, _i64p, _i64p, _i64, _i64, _i64]
                                  + [_int] * 6 + [_vp] * 10 + [ctypes.c_size_t, _vp]),
    "mi355_sage_quant_qk_norm_rope_bf16": (_int, [_vp, _vp] + [_int] * 5 + [ctypes.c_float, _i64p, _i64p, _i64, _i64]
                                           + [_vp, _vp, ctypes.c_float, _vp, _vp, _i64, _int]
                                           + [_int] * 3 + [_vp] * 8 + [ctypes.c_size_t, _vp]),
    "mi355_sage_sdpa_bf16_norm_rope": (_int, [_vp] * 4 + [_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [_i64] * 4
                                       + [_int, _vp, _int, _int, _int, _int]
                                       + [_vp, _vp, ctypes.c_float, _vp, _vp, _i64, _int] + [_vp, ctypes.c_size_t]),
    "mi355_sage_sdpa_bf16_norm_rope_train_fwd": (_int, [_vp] * 5 + [_int] * 5 + [ctypes.c_float] + [_i64p] * 4 + [_i64] * 5
                                                 + [_int, _int, _int, _vp, _int]
                                                 + [_vp, _vp, ctypes.c_float, _vp, _vp, _i64, _int] + [_vp, ctypes.c_size_t]),
    "mi355_sage_quant_v_f16": (_int, [_vp] + [_int] * 4 + [_i64p, _i64, _int, _int, _vp, _vp]),
    "mi355_sage_quant_v_fp8": (_int, [_vp] + [_int] * 4 + [_i64p, _i64, _int, _int, _vp, _vp, _vp, ctypes.c_size_t, _vp]),
    "mi355_sage_attn_fwd": (_int, [_vp, _vp, _int, _vp, _vp, _int, _vp, _vp, _int] + [_int] * 8
                            + [_vp, _i64p, _i64, _vp, _vp, _vp]),
    "mi355_sage_attn_fwd_q16": (_int, [_vp, _i64p, _i64, _vp, _int, _vp, _vp, _int, _vp, _vp, _int] + [_int] * 8
                                + [_vp, _i64p, _i64, _vp]),
    "mi355_sage_attn_split_faults": (_int, [_int]),
    "mi355_sage_attn_split_rule": (_int, [_int] * 6),
    "mi355_sage_set_attn_split": (_int, [_int]),
    "mi355_sage_set_attn_split_wait": (_int, [_int]),
    "mi355_sage_version": (ctypes.c_char_p, []),
}

K_SMOOTH = 1
K_BALANCE = 2
ROPE_INTERLEAVED = 0
ROPE_HALFSPLIT = 1
ROPE_TABLES_BF16 = 2
NORM_FULL_ROW = 4

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libmi355_sage.so is not built (%s). Build it with `make -C mojodiffusion_amd/csrc` "
                "or `python -c 'import __graft_entry__ as g; g.build()'`; there is no fallback path." % LIB_PATH)
        # torch ships its own copy of the HIP runtime.  It has to be in the process before this
        # library is loaded, so that the library binds to that same copy: two HIP runtimes in one
        # process cannot both initialise the device (the second reports "no ROCm-capable device").
        import torch  # noqa: F401
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)          # AttributeError if a declared symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def strides_bhnd(n_eff, h, dh):
    """Element strides describing [B, n_eff, H, Dh] contiguous memory as logical
    [B, H, N, D]: {n_eff*H*Dh, Dh, H*Dh, 1} (serenitymojo/ops/attention_flash.mojo:46-54)."""
    return (ctypes.c_int64 * 4)(n_eff * h * dh, dh, h * dh, 1)


def stats_strides(n_q, h):
    """[B, H, N_q, 1] strides {H*N_q, N_q, 1, 1} (attention_flash.mojo:57-65)."""
    return (ctypes.c_int64 * 4)(h * n_q, n_q, 1, 1)
