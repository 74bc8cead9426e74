"""GPU: the C++ statement of the call surface (include/mi355_sage_host.hpp) against the Python one.

tests/cpp/host_mirror_check.cpp — a plain C++ program linked against libmi355_sage.so, no Python
and no torch in the process — fills its tensors from the reference gate's LCG
(serenitymojo/ops/tests/sdpa_flash_parity.mojo:46-53), calls every entry point of the header and
checks its error texts itself; this test runs it, then makes the same calls through
mojodiffusion_amd.attention_sage and demands the same bits."""
import os
import struct
import subprocess

import numpy as np
import pytest
import torch

from mojodiffusion_amd import attention_sage as A
from test_gpu_gate import _pattern

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "mojodiffusion_amd", "lib", "host_mirror_check")


def _records(path):
    out = {}
    with open(path, "rb") as f:
        while True:
            head = f.read(40)
            if len(head) < 40:
                break
            name = head[:32].split(b"\0", 1)[0].decode()
            (n,) = struct.unpack("<Q", head[32:])
            out[name] = np.frombuffer(f.read(n), dtype=np.uint8)
    return out


def _bits(t):
    return t.contiguous().view(torch.uint8).cpu().numpy().reshape(-1)


def test_cpp_host_mirror_gives_the_python_mirrors_bits(tmp_path):
    assert os.path.exists(EXE), "build the library first (make -C mojodiffusion_amd/csrc)"
    path = str(tmp_path / "out.bin")
    run = subprocess.run([EXE, path], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and "host_mirror_check: ok" in run.stdout, (run.returncode, run.stdout[-3000:], run.stderr[-3000:])
    got = _records(path)

    B, S, Skv, H, Dh, N_TXT, REAL_TXT, REAL_LEN = 1, 384, 520, 6, 128, 96, 61, 300
    scale = float(np.float32(0.08838834764831845))
    mk = lambda n, seed, amp, shape: torch.from_numpy(_pattern(n, seed, amp)).to(torch.bfloat16).reshape(shape).cuda()
    nq, nk = B * S * H * Dh, B * Skv * H * Dh
    q, k, v, g = (mk(nq, s, 1.0, (B, S, H, Dh)) for s in (11, 22, 33, 44))
    k2, v2 = (mk(nk, s, 1.0, (B, Skv, H, Dh)) for s in (55, 66))
    mask = mk(B * H * S * Skv, 77, 3.0, (B, H, S, Skv))

    want = {}
    fwd = A.sdpa_flash_train_fwd(q, k, v, scale)
    want["train_fwd.o"], want["train_fwd.stats"] = fwd.o, fwd.stats
    gr = A.sdpa_flash_backward(fwd, g, scale)
    want["bwd.d_q"], want["bwd.d_k"], want["bwd.d_v"] = gr.d_q, gr.d_k, gr.d_v
    want["bwd_dispatch.d_k"] = A.sdpa_flash_backward_dispatch(fwd.q_pad, fwd.k_pad, fwd.v_pad, fwd.o_pad, fwd.stats, g, scale, B, S, H, Dh).d_k
    rect = A.sdpa_flash_train_fwd_rect(q, k2, v2, scale)
    want["rect.o"], want["rect.stats"] = rect.o, rect.stats
    pad = A.sdpa_flash_fwd_padmask(q, k, v, REAL_LEN, scale)
    want["padmask.o"] = pad.o
    want["padmask.d_v"] = A.sdpa_flash_backward(pad, g, scale, real_len=REAL_LEN).d_v
    want["nomask.o"] = A.sdpa_nomask(q, k, v, scale)
    want["nomask_fp8.o"] = A.sdpa_nomask(q, k, v, scale, A.PV_FP8)
    want["tiled.o"] = A.sdpa_nomask_tiled(q, k, v, scale)
    want["cross.o"] = A.sdpa_cross_nomask(q, k2, v2, scale)
    want["keymask.o"] = A.sdpa_qwen_keymask(q, k, v, N_TXT, REAL_TXT, scale)
    want["cross_masked.o"] = A.sdpa_cross_masked(q, k2, v2, mask, scale)
    torch.cuda.synchronize()
    assert sorted(got) == sorted(want)
    for name, t in want.items():
        if name == "padmask.o":
            # rows at and beyond the real length are computed and meaningless in both; compare the real ones
            a = got[name].reshape(B, S, H * Dh * 2)[:, :REAL_LEN]
            b = _bits(t).reshape(B, S, H * Dh * 2)[:, :REAL_LEN]
            assert np.array_equal(a, b), name
            continue
        assert np.array_equal(got[name], _bits(t)), name
