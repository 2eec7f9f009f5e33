"""The build-time guards of ops-transformer_amd/build.py around the LDS-DMA kernels: the compiler pin, the check that, in
the device assembly, m0 is written only as the first half of an (s_mov_b32 m0, global_load_lds_dwordx4) pair, and the
check of the generated code for scratch use, generic memory instructions and merged multiply-convert instructions."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def build():
    spec = importlib.util.spec_from_file_location("ops_transformer_amd_build",
                                                  os.path.join(ROOT, "ops-transformer_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


GOOD = """
_Zkernel:                               ; @kernel
	s_load_dwordx2 s[0:1], s[4:5], 0x0
	v_readfirstlane_b32 s12, v3
	s_mov_b32 m0, s12
	global_load_lds_dwordx4 v5, s[2:3]
	s_cmp_eq_u32 m0, 0                  ; reading m0 is no write
	s_mov_b32 m0, s13
	global_load_lds_dwordx4 v6, s[2:3] nt
	s_endpgm
"""


def _write(tmp_path, text):
    p = tmp_path / "k.s"
    p.write_text(text)
    return str(p)


def test_assembly_guard_accepts_glued_pairs(build, tmp_path):
    assert build.check_lds_dma_assembly(_write(tmp_path, GOOD)) == 2


@pytest.mark.parametrize("bad", [
    GOOD.replace("\ts_mov_b32 m0, s13\n", "\ts_mov_b32 m0, s13\n\ts_nop 0\n"),           # something between the two
    GOOD.replace("\ts_mov_b32 m0, s13\n", ""),                                            # a load without its m0 write
    GOOD.replace("\ts_endpgm", "\ts_add_u32 m0, s1, s2\n\ts_endpgm"),                     # m0 written for another purpose
    GOOD.replace("\ts_endpgm", "\ts_mov_b32 m0, s1\n\tds_gws_init v0 gds\n\ts_endpgm"),   # m0 for a non-DMA user
    "\ts_endpgm\n",                                                                       # no LDS-DMA load at all
])
def test_assembly_guard_refuses_anything_else(build, tmp_path, bad):
    with pytest.raises(RuntimeError):
        build.check_lds_dma_assembly(_write(tmp_path, bad))


def test_compiler_pin(build, monkeypatch):
    assert any(tag in build.check_compiler() for tag in build.VALIDATED_COMPILERS)  # this image's compiler is the validated one
    monkeypatch.setattr(build, "compiler_version", lambda: "AMD clang version 99.0.0git (roc-99.0.0)")
    monkeypatch.delenv("OPAPI_ALLOW_UNVALIDATED_COMPILER", raising=False)
    with pytest.raises(RuntimeError, match="validated"):
        build.check_compiler()
    monkeypatch.setenv("OPAPI_ALLOW_UNVALIDATED_COMPILER", "1")
    assert "roc-99" in build.check_compiler()


CODEGEN_GOOD = """
_ZN4gemm16StreamGemmKernelILi1ELi0EEEvv:
	v_mul_f32_e32 v1, v2, v3
	v_cvt_f16_f32_e32 v1, v1
	global_load_dword v4, v[0:1], off
	s_endpgm
	.amdhsa_kernel _ZN4gemm16StreamGemmKernelILi1ELi0EEEvv
		.amdhsa_private_segment_fixed_size 0
		.amdhsa_next_free_vgpr 132
	.end_amdhsa_kernel
	.amdhsa_kernel _ZN4gemm13RequantKernelEv
		.amdhsa_private_segment_fixed_size 0
	.end_amdhsa_kernel
"""


def test_codegen_guard_accepts_clean_kernels(build, tmp_path):
    assert build.check_ring_kernel_codegen(_write(tmp_path, CODEGEN_GOOD)) == 1


@pytest.mark.parametrize("bad", [
    CODEGEN_GOOD.replace(".amdhsa_private_segment_fixed_size 0\n\t\t.amdhsa_next", ".amdhsa_private_segment_fixed_size 48\n\t\t.amdhsa_next"),  # a ring kernel spills
    CODEGEN_GOOD.replace("v_cvt_f16_f32_e32 v1, v1", "v_fma_mixlo_f16 v1, v2, v3, 0"),       # product and conversion merged
    CODEGEN_GOOD.replace("global_load_dword v4, v[0:1], off", "flat_load_dword v4, v[0:1]"),  # a generic load
    CODEGEN_GOOD.replace("StreamGemmKernel", "OtherKernel"),                                  # nothing to check
])
def test_codegen_guard_refuses(build, tmp_path, bad):
    assert bad != CODEGEN_GOOD
    with pytest.raises(RuntimeError):
        build.check_ring_kernel_codegen(_write(tmp_path, bad))
