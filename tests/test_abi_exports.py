"""CPU-side checks of the C ABI: the shared library loads without a GPU and
exports every function include/mi355_sage.h declares; argument validation that
needs no device returns the documented codes."""
import ctypes
import os
import re

from mojodiffusion_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions(header="mi355_sage.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_sage_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared_functions()
    assert len(names) >= 12
    test_names = _declared_functions("mi355_sage_test.h")         # the library's own test switches
    assert test_names and not set(test_names) & set(names)
    L = ctypes.CDLL(_lib.LIB_PATH)
    for n in names + test_names:
        assert hasattr(L, n), "library does not export %s" % n
    assert sorted(_lib.SIGNATURES) == sorted(names + test_names)  # the Python binding covers both headers


def test_no_gpu_helpers():
    L = _lib.lib()
    assert L.mi355_sage_version().startswith(b"mi355_sage")
    assert L.mi355_sage_pad_q(1) in (128, 256) and L.mi355_sage_pad_q(4608) == 4608
    assert L.mi355_sage_pad_kv(32760) == 32768
    for variant in (0, 1):
        slots = sorted(L.mi355_sage_v_slot(k, variant) for k in range(64))
        assert slots == list(range(64))            # a permutation of the tile
    assert L.mi355_sage_v_slot(64, 0) == -1
    assert L.mi355_sage_workspace_bytes(1, 24, 4608, 4608, 128, 0) > 3 * 24 * 4608 * 128
    assert L.mi355_sage_workspace_bytes(1, 24, 4608, 4608, 96, 0) == 0
    assert L.mi355_sage_workspace_bytes(0, 24, 4608, 4608, 128, 0) == 0


def test_split_schedule_is_a_function_of_the_shape():
    """Hand-over slots (256 workgroups x (D/32*16 + 2) x 512 floats + 4 KiB of flags) are part of the
    workspace exactly for the shapes that split: fp16 variant, more than 256 row tiles, last round of
    256 at most half full, 16 % or more of the launch idle, spans of 16 steps or more.  The size is a
    function of the shape alone: the test switch that forces a schedule does not move it."""
    L = _lib.lib()
    rule = lambda B, H, S, D, variant=0: L.mi355_sage_attn_split_rule(B, H, S, S, D, variant)
    assert rule(1, 33, 2048, 64) == 256          # 264 tiles: 1.03 rounds
    assert rule(1, 19, 4352, 128) == 256         # 323 tiles
    assert rule(1, 32, 4608, 128) == 256         # 576 tiles: 2.25 rounds
    assert rule(1, 24, 4608, 128) == 0           # 432 tiles: last round 69 % full
    assert rule(2, 30, 4352, 128) == 0           # 1020 tiles: 3.98 rounds
    assert rule(1, 24, 16896, 128) == 0          # 1584 tiles: idle share 12 %
    assert rule(1, 32, 1536, 128) == 0           # 192 tiles: fewer than compute units
    assert rule(1, 8, 1024, 64) == 0
    assert rule(1, 32, 4608, 128, 1) == 0        # the e4m3 variant keeps one workgroup per row tile
    assert rule(1, 32, 4608, 256) == 0           # so do 256 channels
    slots = lambda D: 4096 + 256 * ((D // 32) * 16 + 2) * 512 * 4
    # same tensors, one shape that splits and one that does not: the difference is the slots
    # (items and key tiles decide; 2 x 16 heads of 4608 rows are 576 row tiles like 1 x 32 heads)
    assert L.mi355_sage_workspace_bytes(1, 32, 4608, 4608, 128, 0) - L.mi355_sage_workspace_bytes(1, 32, 4608, 4608, 128, 1) \
        == slots(128) + (L.mi355_sage_workspace_bytes(1, 24, 4608, 4608, 128, 0) - L.mi355_sage_workspace_bytes(1, 24, 4608, 4608, 128, 1)) * 32 // 24
    before = L.mi355_sage_workspace_bytes(1, 2, 512, 512, 64, 0)
    assert L.mi355_sage_set_attn_split(64) == 0
    try:
        assert L.mi355_sage_workspace_bytes(1, 2, 512, 512, 64, 0) == before
    finally:
        L.mi355_sage_set_attn_split(0)
    for bad in (-2, 12, 1032):
        assert L.mi355_sage_set_attn_split(bad) == -1


def test_argument_validation_without_device():
    """Order and codes of serenitymojo/ops/cshim/cudnn_sdpa.cpp:391-393: null
    pointers, non-positive dims, null strides -> -1 before anything touches a GPU.
    The pointers below are not memory: every call here has to be refused by the argument checks,
    which run before the first HIP call.  Where a device is present the test does not run at all
    (tests/test_gpu_attn.py holds the same refusals with real buffers there), so that no change of
    a limit can turn one of these calls into a launch on a made-up address."""
    import pytest
    import torch
    if torch.cuda.is_available():
        pytest.skip("made-up pointers: runs only where no device can be reached")
    L = _lib.lib()
    st = _lib.strides_bhnd(128, 2, 128)
    fake = ctypes.c_void_p(4096)
    ok_dims = (1, 2, 128, 128, 128)
    call = lambda q, k, v, o, dims, s0: L.mi355_sage_sdpa_bf16(
        q, k, v, o, *dims, 0.1, s0, st, st, st, 0, 0, 0, 0, 0, None, 0, None, 0)
    assert call(None, fake, fake, fake, ok_dims, st) == -1
    assert call(fake, fake, fake, None, ok_dims, st) == -1
    assert call(fake, fake, fake, fake, (1, 0, 128, 128, 128), st) == -1
    assert call(fake, fake, fake, fake, (1, 2, 128, -4, 128), st) == -1
    assert call(fake, fake, fake, fake, ok_dims, None) == -1
    # unsupported configurations -> -2
    assert L.mi355_sage_sdpa_bf16(fake, fake, fake, fake, 1, 2, 128, 128, 96, 0.1, st, st, st, st,
                                  0, 0, 0, 0, 0, None, 0, None, 0) == -2          # head dim
    assert L.mi355_sage_sdpa_bf16(fake, fake, fake, fake, 1, 2, 128, 128, 128, 0.1, st, st, st, st,
                                  0, 0, 0, 0, 0, None, 7, None, 0) == -2          # variant
    bad = (ctypes.c_int64 * 4)(128 * 2 * 128, 128, 2 * 128, 2)
    assert L.mi355_sage_sdpa_bf16(fake, fake, fake, fake, 1, 2, 128, 128, 128, 0.1, bad, st, st, st,
                                  0, 0, 0, 0, 0, None, 0, None, 0) == -2          # strided head dim
    assert L.mi355_sage_sdpa_bf16(fake, fake, fake, fake, 1, 2, 128, 128, 128, 0.1, st, st, st, st,
                                  3, 0, 0, 0, 0, None, 0, None, 0) == -2          # misaligned offset
    n_long = 4096 * 64 + 1                            # one key more than 4096 scale blocks of 64 tokens
    st_long = _lib.strides_bhnd(n_long, 2, 128)
    assert L.mi355_sage_sdpa_bf16(fake, fake, fake, fake, 1, 2, 128, n_long, 128, 0.1, st, st_long, st_long, st,
                                  0, 0, 0, 0, 0, None, 0, None, 0) == -2          # more K scale blocks than the kernel stages
    # workspace too small -> -3 (checked before any launch)
    assert L.mi355_sage_sdpa_bf16(fake, fake, fake, fake, 1, 2, 128, 128, 128, 0.1, st, st, st, st,
                                  0, 0, 0, 0, 0, None, 0, ctypes.c_void_p(256 * 64), 1024) == -3
    assert L.mi355_sage_sdpa_bf16_train_fwd(fake, fake, fake, fake, None, 1, 2, 128, 128, 128, 0.1, st, st, st, st,
                                            0, 0, 0, 0, 0, 0, 128, 128, None, 0, None, 0) == -1   # Stats null


def test_host_mirror_error_strings():
    import pytest
    import torch
    from mojodiffusion_amd import attention_sage as A
    q = torch.zeros((1, 128, 2, 64), dtype=torch.float32)
    with pytest.raises(A.Error, match="q/k/v must be BF16"):
        A.sdpa_flash_train_fwd(q, q, q, 0.1)
    with pytest.raises(A.Error, match="sdpa_nomask: q/k/v dtype mismatch"):
        A.sdpa_nomask(q, q.to(torch.bfloat16), q, 0.1)
    with pytest.raises(A.Error, match=r"sdpa_nomask: q must be rank-4 \[B,S,H,Dh\]"):
        A.sdpa_nomask(q[0], q[0], q[0], 0.1)
    qb = torch.zeros((1, 100, 2, 64), dtype=torch.bfloat16)
    with pytest.raises(A.Error, match="S_BUF must be 128-aligned"):
        A.sdpa_flash_fwd_padmask(qb, qb, qb, 50, 0.1)
    qb = torch.zeros((1, 128, 2, 64), dtype=torch.bfloat16)
    with pytest.raises(A.Error, match=r"real_len out of \[1, S_BUF\]"):
        A.sdpa_flash_fwd_padmask(qb, qb, qb, 0, 0.1)
    with pytest.raises(A.Error, match="no CPU fallback"):
        A.sdpa_nomask(qb, qb, qb, 0.1)
    with pytest.raises(A.Error, match="sdpa_nomask_tiled: q/k/v dtype mismatch"):
        A.sdpa_nomask_tiled(q, qb, q, 0.1)
    with pytest.raises(A.Error, match="sdpa: q/mask dtype mismatch"):
        A.sdpa(qb, qb, qb, torch.zeros((1, 2, 128, 128)), 0.1)
    with pytest.raises(A.Error, match=r"sdpa: mask must be \[B,H,S,S\]"):
        A.sdpa(qb, qb, qb, torch.zeros((1, 2, 128, 64), dtype=torch.bfloat16), 0.1)
    with pytest.raises(A.Error, match=r"sdpa_cross_masked: mask must be \[B,H,Sq,Skv\]"):
        A.sdpa_cross_masked(qb[:, :64], qb, qb, torch.zeros((1, 2, 128, 128), dtype=torch.bfloat16), 0.1)
    with pytest.raises(A.Error, match="sdpa_chunked: q/k/v dtype mismatch"):
        A.sdpa_chunked(q, qb, q, torch.zeros((1, 2, 128, 128)), 0.1)
    with pytest.raises(A.Error, match="sdpa_qwen_keymask: real_txt_len out of range"):
        A.sdpa_qwen_keymask(qb, qb, qb, 64, 65, 0.1)
    with pytest.raises(A.Error, match="sdpa_qwen_keymask: N_TXT must be <= S"):
        A.sdpa_qwen_keymask(qb, qb, qb, 129, 5, 0.1)
    with pytest.raises(A.Error, match="sdpa_qwen_keymask: k/v shape mismatch"):
        A.sdpa_qwen_keymask(qb, qb[:, :64], qb, 64, 5, 0.1)


def test_header_is_plain_c_and_links_from_c(tmp_path):
    """include/mi355_sage.h is the boundary a Mojo / C / C++ caller binds: it has to compile as
    strict C11 and as C++ with nothing but the standard headers, and a C program linked against
    the library has to resolve its symbols (no torch, no Python in between)."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None or shutil.which("g++") is None:
        import pytest
        pytest.skip("no host compiler")
    inc = os.path.join(ROOT, "include")
    src = tmp_path / "use.c"
    src.write_text(
        '#include "mi355_sage.h"\n'
        '#include <stdio.h>\n'
        '#include <string.h>\n'
        'int main(void) {\n'
        '    /* argument errors are reported before any device is touched */\n'
        '    int rc = mi355_sage_sdpa_bf16(NULL, NULL, NULL, NULL, 1, 1, 1, 1, 128, 1.0f, NULL, NULL, NULL, NULL,\n'
        '                                  0, 0, 0, 0, 0, NULL, MI355_SAGE_PV_FP16, NULL, 0);\n'
        '    if (rc != MI355_SAGE_EINVAL) return 2;\n'
        '    if (strncmp(mi355_sage_version(), "mi355_sage", 10) != 0) return 3;\n'
        '    if (mi355_sage_pad_kv(32760) != 32768) return 4;\n'
        '    if (mi355_sage_workspace_bytes(1, 24, 4608, 4608, 128, MI355_SAGE_PV_FP16) == 0) return 5;\n'
        '    printf("ok\\n");\n'
        '    return 0;\n'
        '}\n')
    subprocess.check_call(["gcc", "-std=c11", "-pedantic", "-Wall", "-Wextra", "-Wstrict-prototypes", "-Werror",
                           "-I", inc, "-fsyntax-only", str(src)])
    cpp = tmp_path / "use.cpp"
    cpp.write_text('#include "mi355_sage.h"\nint main() { return mi355_sage_pad_q(1) > 0 ? 0 : 1; }\n')
    subprocess.check_call(["g++", "-std=c++17", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", inc, "-fsyntax-only", str(cpp)])
    exe = tmp_path / "use"
    libdir = os.path.dirname(_lib.LIB_PATH)
    subprocess.check_call(["gcc", "-std=c11", "-I", inc, str(src), "-o", str(exe), "-L", libdir, "-lmi355_sage",
                           "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"])
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.strip() == "ok", (out.returncode, out.stdout, out.stderr)


def test_cpp_host_header_compiles_with_the_host_compiler(tmp_path):
    """include/mi355_sage_host.hpp (the call surface for compiled callers) needs nothing but the
    C ABI header, the standard library and HIP's runtime API header."""
    import shutil
    import subprocess
    if shutil.which("g++") is None or not os.path.exists("/opt/rocm/include/hip/hip_runtime_api.h"):
        import pytest
        pytest.skip("no host compiler or no HIP headers")
    src = tmp_path / "use.cpp"
    src.write_text('#include "mi355_sage_host.hpp"\n'
                   'int main() { mi355_sage_host::DeviceContext ctx; (void)ctx; return mi355_sage_host::PV_FP8 == 1 ? 0 : 1; }\n')
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"),
                           "-isystem", "/opt/rocm/include", "-fsyntax-only", str(src)])
