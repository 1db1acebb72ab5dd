"""The C-ABI library loads on a CPU-only box, exports every symbol that
include/artk.h declares, and rejects bad arguments with error codes before any
GPU work (no compute call is made here)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "artk.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(artk_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(artk_lib):
    from art_amd import _lib

    names = declared_symbols()
    assert len(names) >= 15
    for n in names:
        assert hasattr(artk_lib, n), f"{n} declared in artk.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes table and header disagree"
    assert artk_lib.artk_abi_version() == 4


def test_argument_errors_have_codes_and_messages(artk_lib):
    from art_amd import _lib

    rc = artk_lib.artk_gemm_nt(None, None, None, 256, 256, 64, 0, None)
    assert rc == _lib.ERR_INVALID_ARGUMENT
    assert b"null" in artk_lib.artk_last_error()
    buf = (C.c_char * 4096)()
    p = (C.addressof(buf) + 15) // 16 * 16
    rc = artk_lib.artk_gemm_nt(p, p, p, 256, 256, 100, 0, None)  # K not a multiple of 64
    assert rc == _lib.ERR_UNSUPPORTED_SHAPE
    rc = artk_lib.artk_logprob_fwd(p, p, p, 0, 100, 30, 1024, 64, p, p, p, 4096, None)  # T % S != 0
    assert rc == _lib.ERR_INVALID_ARGUMENT and b"multiple" in artk_lib.artk_last_error()
    rc = artk_lib.artk_logprob_fwd(p, p, p, 0, 128, 128, 1024, 100, p, p, p, 4096, None)  # H % 64 != 0
    assert rc == _lib.ERR_UNSUPPORTED_SHAPE
    rc = artk_lib.artk_logprob_fwd(p, p, p, 0, 128, 128, 1024, 64, p, p, p, 16, None)  # tiny workspace
    assert rc == _lib.ERR_WORKSPACE_TOO_SMALL
    rc = artk_lib.artk_grpo_loss(p, p, p, p, p, None, 0, 64, 64, 1.5, 0.5, 0.0, p, p, p, 4096, None)
    assert rc == _lib.ERR_INVALID_ARGUMENT  # clip_lo > clip_hi
    rc = artk_lib.artk_lora_linear_fwd(p, p, p, p, None, 2.0, 64, 64, 64, 5, p, p, p, 4096, None)  # rank 5
    assert rc == _lib.ERR_UNSUPPORTED_SHAPE
    rc = artk_lib.artk_lora_linear_fwd(p, p, p, p, p + 8, 2.0, 64, 64, 64, 8, p, p, p, 4096, None)
    assert rc == _lib.ERR_INVALID_ARGUMENT and b"aligned" in artk_lib.artk_last_error()   # misaligned bias
    projs = (_lib.LoraProjStruct * 5)()
    rc = artk_lib.artk_lora_linear_multi_fwd(p, projs, 5, 2.0, 64, 64, p, 4096, None)            # five projections
    assert rc == _lib.ERR_INVALID_ARGUMENT
    for q in projs:
        q.W = q.W_t = q.A = q.B = q.y = q.g = q.xa = q.dA = q.dB = p
        q.out, q.r = 64, 24
    rc = artk_lib.artk_lora_linear_multi_bwd(p, projs, 3, 2.0, 64, 64, p, p, 1 << 30, None)      # ranks add up to 72
    assert rc == _lib.ERR_UNSUPPORTED_SHAPE and b"64" in artk_lib.artk_last_error()
    # gathered MoE rows further than 2 GiB from x
    rc = artk_lib.artk_moe_lora_grouped_fwd(p, p, p, p, p, 2.0, p, p, p, 1 << 20, 4096, 64, 8, 8, p, p, p, 4096, None)
    assert rc == _lib.ERR_UNSUPPORTED_SHAPE and b"2 GiB" in artk_lib.artk_last_error()
    # attention: row length not a multiple of 256, head dimension 96
    rc = artk_lib.artk_attn_plan(p, p, 1000, p, 1 << 20, None)
    assert rc == _lib.ERR_UNSUPPORTED_SHAPE
    rc = artk_lib.artk_attn_fwd(p, p, p, p, 256, 2, 1, 96, 192, 96, 96, 96, 96, 96, 192, 96, 0.1, p, p, p, 4096, None)
    assert rc == _lib.ERR_UNSUPPORTED_SHAPE and b"head dimension" in artk_lib.artk_last_error()


def test_check_raises(artk_lib):
    import pytest

    from art_amd import _lib

    artk_lib.artk_gemm_nt(None, None, None, 1, 1, 64, 0, None)
    with pytest.raises(ValueError, match="artk error -1"):
        _lib.check(-1)
    _lib.check(0)


def test_workspace_sizes_are_monotone(artk_lib):
    a = artk_lib.artk_grpo_fused_workspace_bytes(4096, 152064, 3584, 4096)
    b = artk_lib.artk_grpo_fused_workspace_bytes(16384, 152064, 3584, 4096)
    c = artk_lib.artk_grpo_fused_workspace_bytes(16384, 152064, 3584, 2048)
    assert 0 < c < b and a <= b
    assert artk_lib.artk_logprob_fwd_workspace_bytes(16384, 152064, 3584) > 16384 * 1188 * 8


def test_header_is_plain_c(tmp_path):
    """include/artk.h is the C-ABI: it must compile as C99 without any C++ or HIP header."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler here")
    src = tmp_path / "use_header.c"
    src.write_text('#include "artk.h"\nint main(void) { return (int)artk_abi_version(); }\n')
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    r = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, "-fsyntax-only",
                        str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
