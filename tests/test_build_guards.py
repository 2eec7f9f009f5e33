"""The two build-time guards of ops-transformer_amd/build.py around the LDS-DMA kernels: the compiler pin and the check
that, in the device assembly, m0 is written only as the first half of an (s_mov_b32 m0, global_load_lds_dwordx4) pair."""
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
