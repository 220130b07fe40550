"""The C-ABI shared library: it loads, exports every symbol include/flux_hip.h declares, the ctypes
structures have the sizes the header's structs have, and argument checks reject bad input before
any launch (no GPU needed for any of this)."""
import ctypes
import os
import re
import subprocess

import pytest

from triton_kernels import _native as nv

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flux_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(flux_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built():
    assert os.path.exists(nv.lib_path()), "run `python __graft_entry__.py build` first"


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_functions()
    assert len(names) >= 12
    handle = ctypes.CDLL(nv.lib_path())
    for name in names:
        assert hasattr(handle, name), f"{name} is declared in flux_hip.h but not exported"
    assert set(names) == set(nv.SIGNATURES), "ctypes binding table and header disagree"
    assert nv.lib().flux_abi_version() == 4


def test_struct_layouts_match_the_header(tmp_path):
    src = tmp_path / "sizes.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "flux_hip.h"\n'
        "int main(void){printf(\"%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\\n\", sizeof(flux_src4), sizeof(flux_qkv_prep_args), "
        "sizeof(flux_linear_args), sizeof(flux_attn_args), offsetof(flux_qkv_prep_args, pe), "
        "offsetof(flux_linear_args, act_begin), offsetof(flux_attn_args, sm_scale), sizeof(flux_linear_qk_fusion), "
        "offsetof(flux_linear_qk_fusion, eps), offsetof(flux_linear_args, qk));return 0;}\n")
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = [int(t) for t in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    want = [ctypes.sizeof(nv.Src4), ctypes.sizeof(nv.QkvPrepArgs), ctypes.sizeof(nv.LinearArgs), ctypes.sizeof(nv.AttnArgs),
            nv.QkvPrepArgs.pe.offset, nv.LinearArgs.act_begin.offset, nv.AttnArgs.sm_scale.offset,
            ctypes.sizeof(nv.LinearQKFusion), nv.LinearQKFusion.eps.offset, nv.LinearArgs.qk.offset]
    assert got == want


def test_argument_checks_reject_before_launch():
    lib = nv.lib()
    assert lib.flux_rms_norm(None, None, None, None, 1, 1, 1, 8, 0, 0, 0, 0, 0, 1e-6, None) == -1      # null pointer
    assert b"null" in lib.flux_last_error()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    assert lib.flux_rms_norm(p, p, p, None, 1, 1, 1, 70000, 0, 0, 0, 0, 0, 1e-6, None) == -5            # too wide
    assert b"65536" in lib.flux_last_error()
    assert lib.flux_rms_norm(p, p, p, None, 1, 1, 1, 8, 0, 0, 0, 7, 0, 1e-6, None) == -3                # dtype
    assert lib.flux_rms_norm(p, p, p, None, 0, 1, 1, 8, 0, 0, 0, 0, 0, 1e-6, None) == 0                 # empty: no launch
    assert lib.flux_layer_norm_modulation(p, p, p, p, 1, 1, -2, 8, 0, 1e-6, None) == -2                 # shape
    a = nv.AttnArgs()
    a.B, a.H, a.L, a.D = 1, 1, 8, 48
    assert lib.flux_attention_fwd_bf16(ctypes.byref(a), None) == -6                                     # head dim
    la = nv.LinearArgs()
    assert lib.flux_linear_bf16(ctypes.byref(la), None) == -1
    la.A = la.W = la.Y = p
    la.M, la.N, la.K, la.lda, la.ldw = 4, 4, 16, 8, 16
    assert lib.flux_linear_bf16(ctypes.byref(la), None) == -2                                           # lda < K
    la.lda, la.act = 16, 9
    assert lib.flux_linear_bf16(ctypes.byref(la), None) == -6                                           # activation
    la.act, la.in_act = 0, 7
    assert lib.flux_linear_bf16(ctypes.byref(la), None) == -6                                           # input activation
    la.in_act, la.M, la.ldy = nv.ACT_SILU, 16, 4
    assert lib.flux_linear_bf16(ctypes.byref(la), None) == -6                                           # fused SiLU on more than 8 rows
    assert b"M <= 8" in lib.flux_last_error()
    la.in_act, la.M = 0, 4
    la.flags = 2
    assert lib.flux_linear_bf16(ctypes.byref(la), None) == -6                                           # unknown flag bit
    assert b"flags" in lib.flux_last_error()
    la.flags = nv.LINEAR_SHARED_GPU
    qf = nv.LinearQKFusion()
    qf.q_out = qf.k_out = qf.q_scale = qf.k_scale = qf.pe = p
    qf.heads, qf.seq_len, qf.out_len = 1, 256, 256
    la.qk = ctypes.pointer(qf)
    assert lib.flux_linear_bf16(ctypes.byref(la), None) == -6                                           # qk fusion on a 4 x 4 product
    assert b"qk fusion" in lib.flux_last_error()
    la.qk = None
    la.M = 0
    assert lib.flux_linear_bf16(ctypes.byref(la), None) == 0                                            # empty
    assert lib.flux_silu(p, p, -1, 0, None) == -2
    qa = nv.QkvPrepArgs()
    qa.B, qa.H, qa.Lt, qa.Li, qa.D = 1, 0, 0, 4, 128
    assert lib.flux_qkv_prep(ctypes.byref(qa), None) == -2


# ---- generated-code check of the attention kernel (see csrc/check_attention_isa.py) ----------------
def _isa_checker():
    import importlib.util
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "triton-kernels_amd", "csrc", "check_attention_isa.py")
    spec = importlib.util.spec_from_file_location("check_attention_isa", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_attention_isa_checker_flags_what_it_should(tmp_path):
    chk = _isa_checker()
    good = "\n".join([
        "_ZN4flux19attn_fwd_w64_kernelILi4ELi4EEEvNS_10AttnParamsE:",
        "\tv_add_f32_e32 v1, v2, v3",
        "\t;;#ASMSTART", "\tv_mfma_f32_16x16x32_bf16 a[0:3], v[4:7], v[8:11], a[0:3]", "\t;;#ASMEND",
        "\ts_endpgm"])
    f = tmp_path / "good.s"
    f.write_text(good)
    assert chk.check(str(f)) == []
    for bad_line in ("\tv_accvgpr_write_b32 a5, v1", "\tscratch_store_dword off, v1, off offset:4", "\tds_read_b128 a[4:7], v1"):
        f = tmp_path / "bad.s"
        f.write_text(good.replace("\tv_add_f32_e32 v1, v2, v3", bad_line))
        assert len(chk.check(str(f))) == 1, bad_line
    f = tmp_path / "none.s"
    f.write_text("_Zother:\n\ts_endpgm\n")
    assert chk.check(str(f))  # no instantiation found is an error too


def test_attention_generated_code_uses_no_accumulation_registers_of_its_own():
    """The assembly the build keeps must pass the check (build() makes it; skipped when not built): the
    head-dim-128 and the head-dim-64 instantiation are two translation units."""
    import pytest
    for unit in ("attention", "attention_d64"):
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "build", "csrc", unit + "-hip-amdgcn-amd-amdhsa-gfx950.s")
        if not os.path.exists(path):
            pytest.skip("library not built in this tree")
        assert _isa_checker().check(path) == []


def test_gemm_generated_code_does_not_spill(tmp_path):
    """The tiled GEMM must not touch scratch memory (a spill costs a factor of several in time and nothing
    in correctness): the checker flags a spill, and the assembly the build keeps passes it."""
    import importlib.util
    import pytest
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("check_no_scratch", os.path.join(here, "..", "triton-kernels_amd", "csrc", "check_no_scratch.py"))
    chk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(chk)
    good = "_ZN4flux19gemm_nt_ring_kernelILi4ELb0EEEvNS_10GemmParamsE:\n\tv_add_f32_e32 v1, v2, v3\n\ts_endpgm\n"
    f = tmp_path / "g.s"
    f.write_text(good)
    assert chk.check(str(f), "gemm_nt_ring_kernel") == []
    f.write_text(good.replace("\tv_add_f32_e32 v1, v2, v3", "\tscratch_store_dwordx4 off, v[40:43], off ; 16-byte Folded Spill"))
    assert len(chk.check(str(f), "gemm_nt_ring_kernel")) == 1
    assert chk.check(str(f), "no_such_kernel")
    path = os.path.join(here, "..", "build", "csrc", "gemm_bf16-hip-amdgcn-amd-amdhsa-gfx950.s")
    if not os.path.exists(path):
        pytest.skip("library not built in this tree")
    assert chk.check(path, "gemm_nt_ring_kernel") == []
    assert chk.check(path, "gemm_nt_rect_kernel") == []
